// finalizer_stress.cc -- the adapter's host logic (GPUAllreduce::Execute, GPUOpContext::FinalizeGPUQueue,
// the finalizer ThreadPool, pooled events, callbacks) against the pretend device of fake_hvdhip.cc.
// Meant to be built with -fsanitize=thread: every scenario must come out right AND race-free.
// Prints "finalizer ok" when all scenarios pass.
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <set>
#include <stdexcept>
#include <thread>
#include <vector>

#include "hvd_hip_adapter.h"

using namespace horovod::common;

extern "C" {
void fake_set_kernel_delay_us(int us);
void fake_fail_next_event_syncs(int n);
int fake_events_outstanding();
int fake_set_device_calls_on_other_threads(void);
}

#define REQUIRE(cond)                                                     \
  do {                                                                    \
    if (!(cond)) {                                                        \
      std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
      std::exit(1);                                                       \
    }                                                                     \
  } while (0)

namespace {

double now_s() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

// One response's tensors, outputs, peer buffer and what its callbacks saw.
struct Response {
  std::vector<std::vector<float>> tensors, outputs;
  std::vector<float> peer;  // laid out like the fusion buffer (16-byte padded offsets)
  std::vector<TensorTableEntry> entries;
  std::atomic<int> callbacks{0};
  std::atomic<int> failures{0};
  std::atomic<int> with_event{0};
  double completed_at = 0;
  std::thread::id finished_on;
  std::mutex mu;
  std::string reason;
};

void build(Response& r, int seed, const std::vector<int>& counts) {
  std::srand((unsigned)seed);
  int64_t off = 0;
  std::vector<int64_t> offs;
  for (int c : counts) {
    offs.push_back(off);
    off += 16 * ((c * 4 + 15) / 16);
  }
  r.peer.assign((size_t)off / 4, 0.f);
  for (size_t i = 0; i < counts.size(); ++i) {
    std::vector<float> t((size_t)counts[i]);
    for (auto& x : t) x = (float)(std::rand() % 2001 - 1000) / 64.f;
    for (int j = 0; j < counts[i]; ++j) r.peer[(size_t)offs[i] / 4 + (size_t)j] = (float)(std::rand() % 2001 - 1000) / 32.f;
    r.tensors.push_back(t);
    r.outputs.emplace_back((size_t)counts[i], -1.f);
  }
  r.entries.resize(counts.size());
  for (size_t i = 0; i < counts.size(); ++i) {
    TensorTableEntry& e = r.entries[i];
    e.tensor_name = "r" + std::to_string(seed) + "." + std::to_string(i);
    e.tensor_data = r.tensors[i].data();
    e.output_data = r.outputs[i].data();
    e.num_elements = counts[i];
    e.dtype = HOROVOD_FLOAT32;
    Response* rp = &r;
    e.callback = [rp](const Status& s) {
      if (!s.ok()) {
        ++rp->failures;
        std::lock_guard<std::mutex> g(rp->mu);
        rp->reason = s.reason();
      }
      if (s.event.event) ++rp->with_event;
      {
        std::lock_guard<std::mutex> g(rp->mu);
        rp->completed_at = now_s();
        rp->finished_on = std::this_thread::get_id();
      }
      ++rp->callbacks;
    };
  }
}

void check(const Response& r, const std::vector<int>& counts, float pre, float post, bool with_peer) {
  int64_t off = 0;
  for (size_t i = 0; i < counts.size(); ++i) {
    for (int j = 0; j < counts[i]; ++j) {
      float v = pre == 1.f ? r.tensors[i][(size_t)j] : pre * r.tensors[i][(size_t)j];
      if (with_peer) v = v + r.peer[(size_t)off / 4 + (size_t)j];
      if (post != 1.f) v = post * v;
      REQUIRE(r.outputs[i][(size_t)j] == v);
    }
    off += 16 * ((counts[i] * 4 + 15) / 16);
  }
}

// A fusion buffer as a framework would hand it out: host memory here, counted when it is freed.
std::atomic<int> g_buffers_freed{0};
class HostBuffer : public PersistentBuffer {
public:
  explicit HostBuffer(int64_t size) : mem_((size_t)size) {}
  ~HostBuffer() override { ++g_buffers_freed; }
  const void* AccessData() const override { return mem_.data(); }

private:
  std::vector<char> mem_;
};
std::shared_ptr<PersistentBuffer> allocate_host(int64_t size, int) { return std::make_shared<HostBuffer>(size); }

struct Rig {
  GPUContext context;
  GlobalState state;
  GPUAllreduce* op = nullptr;
  Rig(int slots, int threads, bool async_completion = false, bool elastic = false, bool timeline = false) {
    state.num_nccl_streams = slots;
    state.enable_async_completion = async_completion;
    state.elastic_enabled = elastic;
    state.timeline_initialized = timeline;
    for (int slot = 0; slot < slots; ++slot) {
      Status s = state.fusion_buffer.InitializeBuffer(1 << 20, 0, allocate_host, slot, nullptr, nullptr);
      REQUIRE(s.ok());
    }
    context.streams.resize((size_t)slots);
    if (threads > 0) context.finalizer_thread_pool.create(threads);
    op = new GPUAllreduce(&context, &state);
  }
  ~Rig() {
    context.finalizer_thread_pool.reset();
    delete op;
  }
};

void wait_for(const Response& r) {
  while (r.callbacks.load() < (int)r.entries.size()) std::this_thread::sleep_for(std::chrono::microseconds(50));
}

// 1. Many responses over two slots: results, one callback per entry, all from finalizer threads.
void many_responses() {
  Rig rig(2, 2);
  const std::vector<int> counts = {5, 1000, 3, 257};
  const int n = 300;
  std::vector<Response> rs((size_t)n);
  for (int i = 0; i < n; ++i) build(rs[(size_t)i], i, counts);
  for (int i = 0; i < n; ++i) {
    std::vector<const void*> peers = {rs[(size_t)i].peer.data()};
    Status s = rig.op->Execute(rs[(size_t)i].entries, 0.125, 0.5, peers);
    REQUIRE(s.in_progress());
    REQUIRE(rig.state.current_nccl_stream == (i + 1) % 2);
  }
  rig.context.finalizer_thread_pool.wait_idle();
  std::set<std::thread::id> finishers;
  for (auto& r : rs) {
    REQUIRE(r.callbacks == (int)counts.size() && r.failures == 0 && r.with_event == 0);
    REQUIRE(r.finished_on != std::this_thread::get_id());
    finishers.insert(r.finished_on);
    check(r, counts, 0.125f, 0.5f, true);
  }
  REQUIRE(finishers.size() <= 2);
  REQUIRE(fake_set_device_calls_on_other_threads() >= n);  // SetDevice at the top of every finalizer task
  REQUIRE(fake_events_outstanding() == 0);                 // every pooled event went back
  REQUIRE(rig.op->cached_plans() == (size_t)128);          // 300 distinct entry lists, bounded cache
  std::printf("many responses: %d over 2 slots, %zu finalizer thread(s) saw completions\n", n, finishers.size());
}

// 2. Two consecutive responses on alternating slots are both in flight before either completes, and
//    run side by side on the pretend device.
void two_in_flight() {
  Rig rig(2, 2);
  const std::vector<int> counts = {64, 64};
  std::vector<Response> rs(4);
  for (int i = 0; i < 4; ++i) build(rs[(size_t)i], 1000 + i, counts);
  // warm-up: plans and streams exist afterwards
  for (int i = 0; i < 2; ++i) {
    std::vector<const void*> peers = {rs[(size_t)i].peer.data()};
    rig.op->Execute(rs[(size_t)i].entries, 1.0, 1.0, peers);
  }
  rig.context.finalizer_thread_pool.wait_idle();
  fake_set_kernel_delay_us(20000);  // 3 kernels of 20 ms per response
  const double t0 = now_s();
  double returned[2];
  for (int i = 2; i < 4; ++i) {
    std::vector<const void*> peers = {rs[(size_t)i].peer.data()};
    rig.op->Execute(rs[(size_t)i].entries, 1.0, 1.0, peers);
    returned[i - 2] = now_s();
  }
  REQUIRE(rs[2].callbacks == 0 && rs[3].callbacks == 0);  // neither has completed: both are in flight
  rig.context.finalizer_thread_pool.wait_idle();
  fake_set_kernel_delay_us(0);
  const double total = now_s() - t0;
  REQUIRE(returned[1] < rs[2].completed_at && returned[1] < rs[3].completed_at);
  REQUIRE(returned[1] - t0 < 0.030);  // Execute does not wait for the device
  REQUIRE(total < 0.100);             // 2 x 60 ms of kernels took well under 120 ms: the slots overlapped
  check(rs[2], counts, 1.f, 1.f, true);
  check(rs[3], counts, 1.f, 1.f, true);
  std::printf("two in flight: both Executes returned after %.1f ms, both responses done after %.1f ms\n",
              (returned[1] - t0) * 1e3, total * 1e3);
}

// 3. A failure on the finalizer thread reaches every entry's callback as an error Status.
void failure_reaches_callbacks() {
  Rig rig(1, 1);
  const std::vector<int> counts = {10, 20, 30};
  Response r;
  build(r, 7, counts);
  fake_fail_next_event_syncs(1);
  Status s = rig.op->Execute(r.entries, 1.0, 1.0, {});
  REQUIRE(s.in_progress());
  rig.context.finalizer_thread_pool.wait_idle();
  REQUIRE(r.callbacks == 3 && r.failures == 3);
  REQUIRE(r.reason.find("hipEventSynchronize failed") != std::string::npos);
  // the pool goes on working afterwards
  Response r2;
  build(r2, 8, counts);
  rig.op->Execute(r2.entries, 0.5, 1.0, {});
  rig.context.finalizer_thread_pool.wait_idle();
  REQUIRE(r2.callbacks == 3 && r2.failures == 0);
  check(r2, counts, 0.5f, 1.f, false);
  std::printf("failure: %s\n", r.reason.c_str());
}

// 3b. A response that fails while it is being queued (an unsupported dtype reaches the pack) throws out
//     of Execute, calls no callback, and leaves no pooled event behind.
void failure_while_queueing() {
  Rig rig(1, 1, false, false, /*timeline=*/true);  // the QUEUE event is already in the op's queue when the pack fails
  const std::vector<int> counts = {10, 20};
  Response r;
  build(r, 11, counts);
  for (auto& e : r.entries) e.dtype = HOROVOD_INT32;  // the pretend device packs float32 only
  bool threw = false;
  try {
    rig.op->Execute(r.entries, 1.0, 1.0, {});
  } catch (const std::logic_error&) {
    threw = true;
  }
  rig.context.finalizer_thread_pool.wait_idle();
  REQUIRE(threw && r.callbacks == 0);
  REQUIRE(fake_events_outstanding() == 0);
}

// 4. No finalizer threads: the completion runs on the caller's thread before Execute returns.
void inline_completion() {
  Rig rig(2, 0);
  const std::vector<int> counts = {100, 1};
  Response r;
  build(r, 9, counts);
  std::vector<const void*> peers = {r.peer.data()};
  Status s = rig.op->Execute(r.entries, 1.0, 0.25, peers);
  REQUIRE(s.in_progress());
  REQUIRE(r.callbacks == 2 && r.finished_on == std::this_thread::get_id());
  check(r, counts, 1.f, 0.25f, true);
}

// 5. Asynchronous completion: nothing is waited for; the callbacks get an event that has been
//    recorded behind the response, and the event is released after them.
void async_completion() {
  Rig rig(1, 1, /*async_completion=*/true);
  const std::vector<int> counts = {50, 60};
  Response r;
  build(r, 10, counts);
  fake_set_kernel_delay_us(5000);
  rig.op->Execute(r.entries, 0.5, 1.0, {});
  rig.context.finalizer_thread_pool.wait_idle();
  fake_set_kernel_delay_us(0);
  REQUIRE(r.callbacks == 2 && r.with_event == 2 && r.failures == 0);
  REQUIRE(fake_events_outstanding() == 0);
  rig.context.StreamSynchronize(rig.context.streams[0][0]);
  check(r, counts, 0.5f, 1.f, false);
}

// 6. Elastic polling and the timeline's per-stage events, completed on finalizer threads.
void elastic_and_timeline() {
  Rig rig(2, 2, false, /*elastic=*/true, /*timeline=*/true);
  const std::vector<int> counts = {33, 44};
  std::vector<Response> rs(6);
  for (int i = 0; i < 6; ++i) {
    build(rs[(size_t)i], 20 + i, counts);
    std::vector<const void*> peers = {rs[(size_t)i].peer.data()};
    rig.op->Execute(rs[(size_t)i].entries, 1.0, 1.0, peers);
  }
  rig.context.finalizer_thread_pool.wait_idle();
  for (auto& r : rs) check(r, counts, 1.f, 1.f, true);
  std::lock_guard<std::mutex> g(rig.state.timeline_mutex);
  REQUIRE(rig.state.timeline_activities.size() == 6 * 4);  // QUEUE, MEMCPY_IN, NCCL_ALLREDUCE, MEMCPY_OUT per response
}

// 7. A pool that is reset with work still queued runs it first; tasks from several producers all run.
void pool_semantics() {
  std::atomic<int> ran{0};
  {
    ThreadPool pool;
    pool.create(3);
    std::vector<std::thread> producers;
    for (int p = 0; p < 4; ++p)
      producers.emplace_back([&] {
        for (int i = 0; i < 500; ++i) pool.execute([&] { ++ran; });
      });
    for (auto& t : producers) t.join();
    pool.execute([&] {
      std::this_thread::sleep_for(std::chrono::milliseconds(5));
      ++ran;
    });
    pool.reset();
    REQUIRE(ran == 2001);
    pool.create(1);  // a pool can be created again after a reset
    pool.execute([&] { ++ran; });
    pool.wait_idle();
    REQUIRE(ran == 2002);
  }
  ThreadPool idle;
  idle.wait_idle();  // no threads: nothing to wait for
}

// 7b. A response in flight keeps the fusion buffer it was packed into: the threshold changes while the
//     pretend device still works on the response (InitializeBuffer lets go of the old buffer and
//     allocates another), and the old one is freed only when the response's finalizer has run.
void fusion_buffer_outlives_its_manager_entry() {
  Rig rig(1, 1);
  const std::vector<int> counts = {400, 9};
  Response r;
  build(r, 40, counts);
  std::vector<const void*> peers = {r.peer.data()};
  int init_calls = 0;
  const int freed_before = g_buffers_freed.load();
  auto old_buffer = rig.state.fusion_buffer.GetBuffer(0, 0)->AccessData();
  fake_set_kernel_delay_us(15000);
  rig.op->Execute(r.entries, 0.5, 1.0, peers);
  fake_set_kernel_delay_us(0);
  // the same threshold again: nothing happens
  REQUIRE(rig.state.fusion_buffer.InitializeBuffer(1 << 20, 0, allocate_host, 0, [&] { ++init_calls; }, [&] { ++init_calls; }).ok());
  REQUIRE(init_calls == 0 && rig.state.fusion_buffer.GetBuffer(0, 0)->AccessData() == old_buffer);
  // another threshold: a new buffer, between the two callbacks
  REQUIRE(rig.state.fusion_buffer.InitializeBuffer(2 << 20, 0, allocate_host, 0, [&] { ++init_calls; }, [&] { ++init_calls; }).ok());
  REQUIRE(init_calls == 2 && rig.state.fusion_buffer.GetBuffer(0, 0)->AccessData() != old_buffer);
  REQUIRE(r.callbacks == 0);                             // the response is still on the pretend device ...
  REQUIRE(g_buffers_freed.load() == freed_before);       // ... and still owns the buffer it was packed into
  rig.context.finalizer_thread_pool.wait_idle();
  REQUIRE(r.callbacks == 2 && r.failures == 0);
  REQUIRE(g_buffers_freed.load() == freed_before + 1);   // freed once its finalizer had run
  check(r, counts, 0.5f, 1.f, true);
  // an allocator that fails is reported, and a slot that was never initialised is an error of the op
  Status s = rig.state.fusion_buffer.InitializeBuffer(4 << 20, 0, [](int64_t, int) { return std::shared_ptr<PersistentBuffer>(); }, 0, nullptr, nullptr);
  REQUIRE(!s.ok() && rig.state.fusion_buffer.GetBuffer(0, 0) == nullptr);
  Response r2;
  build(r2, 41, counts);
  bool threw = false;
  try {
    rig.op->Execute(r2.entries, 1.0, 1.0, {});
  } catch (const std::logic_error& e) {
    threw = std::string(e.what()).find("no fusion buffer") != std::string::npos;
  }
  REQUIRE(threw);
}

// 8. WaitForData: the tensors are produced on another stream (a copy that takes 20 ms) with an event
//    recorded behind it; Execute is called at once with that event as every entry's ready event and
//    must not read the tensors before the producer has written them -- by a stream wait, or, with the
//    timeline on, by polling on the host.
void waits_for_the_producer() {
  for (int timeline = 0; timeline < 2; ++timeline) {
    Rig rig(1, 1, false, false, timeline != 0);
    const std::vector<int> counts = {300, 5};
    Response r;
    build(r, 30 + timeline, counts);
    // what the producer will write; the tensors hold something else until then
    std::vector<std::vector<float>> produced = r.tensors;
    for (auto& t : r.tensors)
      for (auto& x : t) x = -12345.f;
    void* producer = nullptr;
    REQUIRE(hvdhip_set_device(0) == 0);
    REQUIRE(hvdhip_stream_create(&producer) == 0);
    void* ready = nullptr;
    REQUIRE(hvdhip_event_acquire(producer, &ready) == 0);
    fake_set_kernel_delay_us(20000);
    for (size_t i = 0; i < counts.size(); ++i)
      REQUIRE(hvdhip_memcpy_async(r.tensors[i].data(), produced[i].data(), produced[i].size() * 4, HVDHIP_MEMCPY_D2D, producer) == 0);
    fake_set_kernel_delay_us(0);
    REQUIRE(hvdhip_event_record(ready, producer) == 0);
    for (auto& e : r.entries) e.ready_events = {ready};
    rig.op->Execute(r.entries, 0.5, 1.0, {});
    rig.context.finalizer_thread_pool.wait_idle();
    REQUIRE(r.callbacks == 2 && r.failures == 0);
    r.tensors = produced;  // check() reads the inputs from here
    check(r, counts, 0.5f, 1.f, false);
    if (timeline) {
      std::lock_guard<std::mutex> g(rig.state.timeline_mutex);
      REQUIRE(rig.state.timeline_activities.front() == WAIT_FOR_DATA);
    }
    REQUIRE(hvdhip_event_release(producer, ready) == 0);
    REQUIRE(hvdhip_stream_destroy(producer) == 0);
  }
}

// 9. The allgather op's fusion-buffer hooks (ops/collective_operations.cc:200-275): every rank's entries
//    packed at the rank's displacement, then one component per (entry, rank) copied out; ragged first
//    dimensions, an empty component.  Each output must be the ranks' tensors one after the other.
void allgather_hooks() {
  Rig rig(1, 1);
  GPUAllgather op(&rig.context, &rig.state);
  const int ranks = 3, n = 4;
  const int64_t sizes[n][ranks] = {{5, 0, 7}, {100, 3, 1}, {1, 1, 1}, {33, 64, 2}};  // elements of entry e on rank r
  std::vector<std::vector<std::vector<float>>> tensors((size_t)ranks);   // [rank][entry]
  std::vector<std::vector<float>> outputs((size_t)n);
  std::vector<int> recvcounts((size_t)ranks, 0), displ((size_t)ranks, 0);
  std::vector<std::vector<int64_t>> csz((size_t)n, std::vector<int64_t>((size_t)ranks)), cof = csz;
  std::vector<int64_t*> csz_p, cof_p;
  float next = 1.f;
  for (int r = 0; r < ranks; ++r) {
    tensors[(size_t)r].resize((size_t)n);
    for (int e = 0; e < n; ++e) {
      for (int64_t i = 0; i < sizes[e][r]; ++i) tensors[(size_t)r][(size_t)e].push_back(next++);
      recvcounts[(size_t)r] += (int)sizes[e][r];
    }
  }
  for (int e = 0; e < n; ++e) {
    int64_t total = 0;
    for (int r = 0; r < ranks; ++r) {
      csz[(size_t)e][(size_t)r] = sizes[e][r];
      total += sizes[e][r];
    }
    outputs[(size_t)e].assign((size_t)total, -1.f);
    csz_p.push_back(csz[(size_t)e].data());
    cof_p.push_back(cof[(size_t)e].data());
  }
  int* dp = displ.data();
  GPUAllgather::SetDisplacements(recvcounts.data(), dp, ranks);
  REQUIRE(displ[0] == 0 && displ[1] == recvcounts[0] && displ[2] == recvcounts[0] + recvcounts[1]);
  int64_t** cofpp = cof_p.data();
  GPUAllgather::SetEntryComponentOffsets((size_t)n, csz_p.data(), recvcounts.data(), cofpp, ranks);
  REQUIRE(hvdhip_set_device(0) == 0);
  rig.context.StreamCreate(&rig.context.streams[0][0]);
  void* buffer_data = nullptr;
  std::vector<TensorTableEntry> entries((size_t)n);
  for (int r = 0; r < ranks; ++r) {
    for (int e = 0; e < n; ++e) {
      entries[(size_t)e].tensor_data = tensors[(size_t)r][(size_t)e].data();
      entries[(size_t)e].output_data = outputs[(size_t)e].data();
      entries[(size_t)e].num_elements = sizes[e][r];
      entries[(size_t)e].dtype = HOROVOD_FLOAT32;
    }
    op.MemcpyInFusionBuffer(entries, displ.data(), r, 4, buffer_data);
  }
  op.MemcpyOutFusionBuffer(cof_p.data(), csz_p.data(), buffer_data, 4, ranks, entries);
  rig.context.StreamSynchronize(rig.context.streams[0][0]);
  for (int e = 0; e < n; ++e) {
    size_t at = 0;
    for (int r = 0; r < ranks; ++r)
      for (float x : tensors[(size_t)r][(size_t)e]) REQUIRE(outputs[(size_t)e][at++] == x);
    REQUIRE(at == outputs[(size_t)e].size());
  }
}

}  // namespace

int main() {
  std::setvbuf(stdout, nullptr, _IONBF, 0);
  pool_semantics();
  many_responses();
  two_in_flight();
  failure_reaches_callbacks();
  failure_while_queueing();
  inline_completion();
  async_completion();
  elastic_and_timeline();
  fusion_buffer_outlives_its_manager_entry();
  waits_for_the_producer();
  allgather_hooks();
  std::printf("finalizer ok\n");
  return 0;
}
