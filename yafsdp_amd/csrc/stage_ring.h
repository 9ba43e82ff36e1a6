// Staging slots for the per-call pointer / mode arrays of tables with more tensors than fit in the kernel
// arguments: pinned host slot -> device slot -> kernel.  Pure bookkeeping over a small runtime interface (no HIP
// headers), so that the state machine can also be driven by a simulated runtime in a host-only test.
//
// A slot keeps what was staged into it, so a call whose arrays equal a slot's content (the caching allocator hands
// autograd the same addresses step after step) reuses the device copy without copying again.  ev[s] marks the end
// of the last kernel that reads slot s, on whichever stream that ran; every reuse is ordered behind it before it
// re-records the event, so the recorded event always covers every earlier reader and the copy before them.  The host
// never waits: a slot whose last kernel has not finished is not overwritten, and when every slot is in that state the
// call fails with `busy_code`.
//
// RT provides:
//   typedef ... Stream;  typedef ... Event;
//   int stream_wait_event(Stream, Event);                       0 or an error code
//   int event_query(Event);                                     0 = complete, RT::kNotReady, or an error code
//   int memcpy_h2d_async(void* dst, const void* src, size_t n, Stream);
//   int event_record(Event, Stream);
#pragma once
#include <stddef.h>
#include <string.h>

namespace yafsdp {

template <class RT, int RING = 8>
struct StageRing {
  typedef typename RT::Stream Stream;
  typedef typename RT::Event Event;
  static constexpr int kRing = RING;

  size_t stage_bytes = 0;        // size of one slot (what is copied)
  char* h_stage[RING] = {};      // pinned host memory
  char* d_stage[RING] = {};      // device memory
  Event ev[RING] = {};
  bool ev_pending[RING] = {};
  bool filled[RING] = {};        // h_stage[s] / d_stage[s] hold a staged set
  int next = 0;

  // Finds or stages the `used` bytes at `cur`; *slot is the slot whose device copy the caller's kernel may read
  // once it is enqueued on `stream` after this call.  Returns 0, `busy_code`, or an error code of the runtime.
  int acquire(RT& rt, const char* cur, size_t used, Stream stream, int busy_code, int* slot) {
    int s = -1;
    for (int i = 0; i < RING; i++) {
      if (filled[i] && memcmp(h_stage[i], cur, used) == 0) { s = i; break; }
    }
    if (s >= 0) {
      // same arrays as an earlier call: the device copy is reused.  This call's kernel is ordered behind the slot's
      // last reader, whichever stream that ran on (on the device; the host does not wait; a wait for an event of
      // the same stream costs nothing).
      if (ev_pending[s]) {
        const int e = rt.stream_wait_event(stream, ev[s]);
        if (e != 0) return e;
      }
    } else {
      for (int k = 0; k < RING && s < 0; k++) {
        const int i = (next + k) % RING;
        if (ev_pending[i]) {
          const int q = rt.event_query(ev[i]);
          if (q == RT::kNotReady) continue;  // its last kernel (and the copy before it) is still in flight
          if (q != 0) return q;
          ev_pending[i] = false;
        }
        s = i;
      }
      if (s < 0) return busy_code;
      next = (s + 1) % RING;
      memcpy(h_stage[s], cur, used);
      filled[s] = true;
      const int e = rt.memcpy_h2d_async(d_stage[s], h_stage[s], stage_bytes, stream);
      if (e != 0) { filled[s] = false; return e; }
    }
    *slot = s;
    return 0;
  }

  // The kernel that reads `slot` has been enqueued on `stream`.
  int finish(RT& rt, int slot, Stream stream) {
    const int e = rt.event_record(ev[slot], stream);
    if (e != 0) return e;
    ev_pending[slot] = true;
    return 0;
  }

  // The launch after acquire() failed: the slot's content is no longer offered for reuse, and the slot stays
  // ordered behind whatever acquire() enqueued (the event is recorded all the same).  Returns `launch_error`.
  int abandon(RT& rt, int slot, Stream stream, int launch_error) {
    filled[slot] = false;
    if (rt.event_record(ev[slot], stream) == 0) ev_pending[slot] = true;
    return launch_error;
  }
};

}  // namespace yafsdp
