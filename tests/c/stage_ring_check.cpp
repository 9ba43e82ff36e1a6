// Host-only check of the staging slots' state machine (yafsdp_amd/csrc/stage_ring.h) against a simulated runtime.
// Test infrastructure: no GPU, no HIP.
//
// The simulated runtime keeps, per stream, the ordered list of operations enqueued on it (copies into a slot,
// kernels that read a slot, event records, waits) and completes them only when the driver says so.  From that log
// it derives the happens-before relation a real device guarantees (stream order, wait -> the record it waited for,
// and "the host saw this event complete" -> everything issued afterwards) and checks, for every slot:
//   * a kernel that reads the slot happens after the latest copy into it that was issued before the kernel, and that
//     copy carried the arrays the kernel's call asked for;
//   * a copy into the slot happens after every kernel that was issued earlier and reads the slot (it must not
//     overwrite what a queued kernel is still going to read), and after every earlier copy into it.
// A random driver mixes streams, repeated and fresh tensor sets, launch failures and completions.
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <set>
#include <vector>

#include "../../yafsdp_amd/csrc/stage_ring.h"

namespace {

enum OpKind { COPY, KERNEL, RECORD, WAIT };
struct Op {
  OpKind kind;
  int stream;
  int slot;            // COPY / KERNEL
  uint64_t content;    // COPY: what was staged; KERNEL: what its call asked for
  int event;           // RECORD / WAIT
  std::vector<int> deps;  // operations that happen before this one (besides its predecessor on the stream)
  bool done = false;
};

struct Sim {
  typedef int Stream;
  typedef int Event;
  static constexpr int kNotReady = 600;
  std::vector<Op> ops;
  std::vector<std::vector<int>> streams;  // op ids per stream, in order
  std::vector<int> last_record;           // per event: op id of its latest record, -1 if none
  std::set<int> host_knows;               // records the host has seen complete (through event_query)
  int fail_next_copy = 0;

  Sim(int n_streams, int n_events) : streams(n_streams), last_record(n_events, -1) {}

  int push(Op op) {
    const int id = int(ops.size());
    for (int r : host_knows) op.deps.push_back(r);  // the host issued this after it saw r complete
    ops.push_back(op);
    streams[op.stream].push_back(id);
    return id;
  }
  int stream_wait_event(Stream s, Event e) {
    Op op{WAIT, s, -1, 0, e, {}};
    if (last_record[e] >= 0) op.deps.push_back(last_record[e]);
    push(op);
    return 0;
  }
  int event_query(Event e) {
    const int r = last_record[e];
    if (r < 0) return 0;
    if (!ops[r].done) return kNotReady;
    host_knows.insert(r);
    return 0;
  }
  int memcpy_h2d_async(void* dst, const void* src, size_t, Stream s) {
    if (fail_next_copy) { fail_next_copy = 0; return 7; }
    const int slot = int(reinterpret_cast<intptr_t>(dst)) - 1;
    uint64_t content;
    memcpy(&content, src, sizeof(content));
    push(Op{COPY, s, slot, content, -1, {}});
    return 0;
  }
  int event_record(Event e, Stream s) {
    last_record[e] = push(Op{RECORD, s, -1, 0, e, {}});
    return 0;
  }
  void kernel(Stream s, int slot, uint64_t content) { push(Op{KERNEL, s, slot, content, -1, {}}); }

  // completes, in stream order, up to `count` further operations of stream s whose dependencies are done
  void advance(int s, int count) {
    for (int id : streams[s]) {
      if (count == 0) break;
      if (ops[id].done) continue;
      for (int d : ops[id].deps)
        if (!ops[d].done) return;  // blocked: nothing later on this stream may run either
      ops[id].done = true;
      --count;
    }
  }

  // does a happen before b?  (a was issued before b)
  bool before(int a, int b) const {
    std::vector<int> stack{b};
    std::vector<char> seen(ops.size(), 0);
    std::vector<int> pos(ops.size(), -1);
    for (const auto& st : streams)
      for (size_t i = 0; i < st.size(); i++) pos[st[i]] = int(i);
    while (!stack.empty()) {
      const int x = stack.back();
      stack.pop_back();
      if (x == a) return true;
      if (x < a || seen[x]) continue;  // ids grow in issue order: nothing issued before a can depend on it
      seen[x] = 1;
      if (pos[x] > 0) stack.push_back(streams[ops[x].stream][pos[x] - 1]);
      for (int d : ops[x].deps) stack.push_back(d);
    }
    return false;
  }
};

int fail(const char* what, int a, int b) {
  printf("FAIL: %s (operations %d and %d)\n", what, a, b);
  return 1;
}

int check(const Sim& sim, int n_slots) {
  for (int slot = 0; slot < n_slots; slot++) {
    int last_copy = -1;
    std::vector<int> readers_since_copy;
    for (int id = 0; id < int(sim.ops.size()); id++) {
      const Op& op = sim.ops[id];
      if (op.slot != slot) continue;
      if (op.kind == KERNEL) {
        if (last_copy < 0) return fail("a kernel reads a slot that was never staged", id, id);
        if (sim.ops[last_copy].content != op.content) return fail("a kernel reads another call's arrays", last_copy, id);
        if (!sim.before(last_copy, id)) return fail("a kernel is not ordered behind the copy it reads", last_copy, id);
        readers_since_copy.push_back(id);
      } else if (op.kind == COPY) {
        for (int r : readers_since_copy)
          if (!sim.before(r, id)) return fail("a copy may overwrite what a queued kernel still reads", r, id);
        if (last_copy >= 0 && !sim.before(last_copy, id)) return fail("two copies into a slot are not ordered", last_copy, id);
        last_copy = id;
        readers_since_copy.clear();
      }
    }
  }
  return 0;
}

int run(unsigned seed, int n_streams, int n_sets, int steps, int* n_busy, int* n_reuse) {
  srand(seed);
  constexpr int kSlots = 8;
  typedef yafsdp::StageRing<Sim, kSlots> Ring;
  Sim sim(n_streams, kSlots);
  Ring ring;
  static char host[kSlots][16];
  ring.stage_bytes = 16;
  for (int i = 0; i < kSlots; i++) {
    ring.h_stage[i] = host[i];
    ring.d_stage[i] = reinterpret_cast<char*>(intptr_t(i + 1));  // the simulated copy decodes the slot from it
    ring.ev[i] = i;
    memset(host[i], 0, 16);
  }
  for (int step = 0; step < steps; step++) {
    const int s = rand() % n_streams;
    // a tensor set the loop has used before (reuse) or a fresh one
    uint64_t content = (rand() % 4 == 0) ? uint64_t(1000000 + step) : uint64_t(1 + rand() % n_sets);
    char cur[16] = {};
    memcpy(cur, &content, sizeof(content));
    if (rand() % 23 == 0) sim.fail_next_copy = 1;
    const size_t n_before = sim.ops.size();
    int slot = -1;
    const int rc = ring.acquire(sim, cur, 16, s, -7, &slot);
    sim.fail_next_copy = 0;
    if (rc == -7) {
      ++*n_busy;
      if (sim.ops.size() != n_before) return fail("a busy call enqueued something", int(n_before), int(sim.ops.size()));
    } else if (rc == 0) {
      if (sim.ops.size() == n_before || sim.ops.back().kind != COPY) ++*n_reuse;
      if (rand() % 11 == 0) {
        ring.abandon(sim, slot, s, 99);  // the launch failed: no kernel reads the slot
      } else {
        sim.kernel(s, slot, content);
        ring.finish(sim, slot, s);
      }
    }  // any other code: the copy failed, nothing else happened
    // the device makes some progress, on some streams more than on others
    for (int k = 0; k < n_streams; k++)
      if (rand() % 3) sim.advance(k, rand() % 6);
    if (rand() % 40 == 0)
      for (int round = 0; round < 8; round++)
        for (int k = 0; k < n_streams; k++) sim.advance(k, 1000);
  }
  return check(sim, kSlots);
}

}  // namespace

int main() {
  int busy = 0, reuse = 0;
  for (unsigned seed = 1; seed <= 60; seed++) {
    const int n_streams = 1 + seed % 3, n_sets = 2 + seed % 13;
    if (run(seed, n_streams, n_sets, 400, &busy, &reuse)) {
      printf("seed %u, %d streams, %d tensor sets\n", seed, n_streams, n_sets);
      return 1;
    }
  }
  if (busy == 0 || reuse == 0) {
    printf("FAIL: the driver never produced a busy ring (%d) or a reused slot (%d)\n", busy, reuse);
    return 1;
  }
  printf("ok: 60 runs of 400 calls, %d reuses, %d busy returns\nPASS\n", reuse, busy);
  return 0;
}
