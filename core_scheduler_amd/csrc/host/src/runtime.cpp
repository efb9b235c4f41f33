// Tensor handles, events, tasks and the three-stream scheduler of the host API, on HIP.
//
// The scheduling rules are the reference's (src/threading/dynamic_scheduler.cpp:131-217):
// submit() runs inline on the caller; a task body runs under a stream guard chosen by its
// priority (main / assist / comm), first making that stream wait for every input that was
// produced on another stream and has not completed; outputs are stamped with the priority
// and an event; assist and comm tasks wait for the last main task, and the tensors they touch
// are parked until the main stream has been made to wait for them a few main tasks later, so
// the caching allocator cannot hand their memory out early.
#include <ATen/hip/HIPEvent.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <ATen/ops/allclose.h>

#include <atomic>
#include <cstdint>
#include <deque>
#include <exception>
#include <mutex>
#include <optional>
#include <string>
#include <vector>

#include "logger.h"
#include "tensor_impl.h"
#include "threading/dynamic_scheduler.h"
#include "threading/event.h"
#include "threading/scheduler_impl.h"
#include "threading/task_impl.h"
#include "trace_range.h"

namespace cs {
// ------------------------------------------------------------------ events
struct Event::Impl {
  void block() {
    settle();
    event.block(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA());
  }
  void record() {
    static std::atomic<uint64_t> counter{0};
    order = ++counter;
    stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().id();
    owed = false;
    event.record();
  }
  // A record that is made only when somebody needs it.  The scheduler stamps the outputs of a
  // main-lane task with such an event instead of recording one per task: a record is a packet
  // between two kernels that keeps the second from starting under the tail of the first (90 tasks
  // of a GPT-2-small step: 2.19 ms with a record each, 1.92 ms without).  Whoever later waits for
  // the event (another lane, the host) has it recorded on `home` then, at the stream's tail at
  // that moment, which covers the task it stands for and whatever the stream got afterwards.
  void defer(const c10::hip::HIPStreamMasqueradingAsCUDA &on) {
    home = on;
    stream = on.id();
    order = 0;
    owed = true;
  }
  void settle() {
    if (!owed) return;
    static auto *mutex = new std::mutex;  // a waiting thread and a submitting one may both get here
    std::lock_guard<std::mutex> lock{*mutex};
    if (!owed) return;
    c10::hip::HIPStreamGuardMasqueradingAsCUDA guard{*home};
    record();
  }
  [[nodiscard]] bool is_owed() const { return owed; }
  // back to the state of a new event (the pool hands impls out again)
  void clear() {
    owed = false;
    order = 0;
    stream = -1;
  }
  // the stream of the last record(), or the one a deferred record will go to
  c10::StreamId stream = -1;
  // position of the last record() among all records of the process; 0 = never recorded.
  // Two events recorded on one stream complete in this order.
  uint64_t order = 0;
  [[nodiscard]] bool query() {
    settle();
    return event.query();
  }
  void synchronize() {
    settle();
    event.synchronize();
  }

 private:
  // Events here order streams of one device and tell the host that work has finished; the data
  // itself reaches the host through stream-ordered copies.  hipEventReleaseToDevice is the
  // runtime's flag for exactly that: a record releases at device scope, so the stream waits,
  // queries and host synchronisations that the scheduler builds on these events synchronize
  // with the recorded work for every reader on this device, without the write-back to system
  // scope of a default event (which costs the recording stream ~2.7 us here instead of ~0.9 us).
  at::cuda::CUDAEvent event{hipEventDisableTiming | hipEventReleaseToDevice};
  std::optional<c10::hip::HIPStreamMasqueradingAsCUDA> home;
  bool owed = false;
};

namespace {
// Events are recycled: creating one costs a driver call (the reference pools them too,
// src/threading/event.cpp:24-48).
struct EventPool {
  std::mutex mutex;
  std::vector<std::shared_ptr<Event::Impl>> free_list;

  std::shared_ptr<Event::Impl> take() {
    {
      std::lock_guard<std::mutex> lock{mutex};
      if (!free_list.empty()) {
        auto e = std::move(free_list.back());
        free_list.pop_back();
        return e;
      }
    }
    return std::make_shared<Event::Impl>();
  }
  void give(std::shared_ptr<Event::Impl> &&e) {
    e->clear();
    std::lock_guard<std::mutex> lock{mutex};
    free_list.push_back(std::move(e));
  }
};
EventPool &pool() {
  static auto *p = new EventPool;  // never destroyed: events may outlive static teardown order
  return *p;
}
}  // namespace

Event::Event() : impl_{pool().take()} {}
Event::Event(std::shared_ptr<Impl> impl) : impl_{std::move(impl)} {}
Event::~Event() {
  // hand the event back only when this handle is the last owner
  if (impl_ && impl_.use_count() == 1) pool().give(std::move(impl_));
}
void Event::block() const { impl_->block(); }
void Event::record() const { impl_->record(); }
bool Event::query() const { return impl_->query(); }
void Event::synchronize() const { impl_->synchronize(); }
const std::shared_ptr<Event::Impl> &Event::impl() const { return impl_; }

// ----------------------------------------------------------------- tensors
ReadOnlyTensor::ReadOnlyTensor() : impl_{std::make_shared<Impl>()} {}
TensorOptions ReadOnlyTensor::options() const { return impl_->options(); }
IntArrayRef ReadOnlyTensor::sizes() const { return impl_->sizes(); }
int64_t ReadOnlyTensor::size(const int64_t dim) const { return impl_->size(dim); }
int64_t ReadOnlyTensor::numel() const { return impl_->numel(); }
void ReadOnlyTensor::wait() const {
  impl_->settle();  // enqueue what the tensor's value still lacks, then wait for all of it
  impl_->event().synchronize();
}
const std::shared_ptr<ReadOnlyTensor::Impl> &ReadOnlyTensor::impl() const { return impl_; }
void ReadOnlyTensor::reset() { impl_ = std::make_shared<Impl>(); }
void Tensor::wait() const { ReadOnlyTensor::wait(); }
std::ostream &print(std::ostream &stream, const ReadOnlyTensor &tensor, const int64_t linesize) {
  tensor.wait();
  return at::print(stream, tensor.impl()->tensor(), linesize);
}

// ------------------------------------------------------------------- tasks
Task::Task(std::shared_ptr<Impl> impl) : impl_{std::move(impl)} {}
void Task::operator()() const { (*impl_)(); }
const std::shared_ptr<Task::Impl> &Task::impl() const { return impl_; }
void Task::reset() { impl_.reset(); }

// -------------------------------------------------------------- schedulers
int64_t Scheduler::get_device_rank() const { return impl_->device_rank(); }
void Scheduler::Impl::submit(Task &&task) {
  CS_ASSERT_TRUE(false, "Scheduler::Impl::submit has no implementation; use DynamicScheduler");
}

namespace {
using Stream = c10::hip::HIPStreamMasqueradingAsCUDA;
using Priority = Task::Impl::Priority;

struct Parked {
  int countdown;                    // main tasks left before the main stream waits for `done`
  Event done;                       // recorded on the side stream after the task
  std::vector<at::Tensor> keep;     // everything the task touched
};

constexpr int kAssistGap = 2;  // the reference's assist_task_gap / comm_task_gap
constexpr int kCommGap = 5;

struct ThreeStreamScheduler final : Scheduler::Impl {
  explicit ThreeStreamScheduler(const int local_rank) : Impl{local_rank} {
    streams_.reserve(Priority::kNumPriority);
    for (int i = 0; i < Priority::kNumPriority; ++i)
      streams_.push_back(c10::hip::getStreamFromPoolMasqueradingAsCUDA(
          /*isHighPriority=*/false, static_cast<c10::DeviceIndex>(local_rank)));
  }

  void submit(Task &&task) override {
    // one submission at a time: the lanes' bookkeeping below is not shared between threads
    // otherwise (the reference's submit is a push into a locked queue)
    std::lock_guard<std::recursive_mutex> lock{submit_mutex_};
    c10::hip::HIPGuardMasqueradingAsCUDA device_guard{static_cast<c10::DeviceIndex>(device_rank_)};
    const auto &body = *task.impl();
    if (body.type() == Task::Impl::kConfig) {
      task();
      return;
    }
    const Priority lane = body.priority();
    c10::hip::HIPStreamGuardMasqueradingAsCUDA stream_guard{streams_[lane]};
    if (lane == Priority::kMain) {
      try {
        age(assist_);
        age(comm_);
        replace(main_done_, run(task, lane));
      } catch (const std::exception &e) {
        CS_ASSERT_TRUE(false, std::string("Task ") + body.name() + " failed with error: " + e.what());
      }
      return;
    }
    wait_for(lane, main_done_);
    Parked parked{lane == Priority::kAssist ? kAssistGap : kCommGap, run(task, lane), touched(body)};
    (lane == Priority::kAssist ? assist_ : comm_).push_front(std::move(parked));
  }

 private:
  // `slot` becomes another handle of `stamp`; the event it held goes back to the pool if this
  // was its last handle
  static void replace(Event &slot, const Event &stamp) {
    const Event old{slot};
    slot = stamp;
  }
  // Make the current stream wait for inputs from other streams, run, stamp the outputs.  One
  // event is recorded per task (the reference records one per output tensor,
  // src/threading/dynamic_scheduler.cpp:150-160): every output, and the caller's own
  // bookkeeping, share it, since each record is a packet the stream has to work through.
  Event run(const Task &task, const Priority lane) {
    // tensors whose last launches were put off get them now, before the body reads or rewrites them
    for (const auto &t : task.impl()->input()) t.impl()->settle();
    for (const auto &t : task.impl()->output()) t.impl()->settle();
    // of the inputs that other streams produced, the one stamped last per stream is waited for:
    // a stream finishes its events in the order it recorded them, so that wait covers the rest
    // (each wait is a packet that stalls this stream for microseconds even when it is granted)
    const c10::StreamId here = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().id();
    constexpr int kMostStreams = 8;
    const Event *latest[kMostStreams] = {};
    int n_latest = 0;
    for (const auto &t : task.impl()->input()) {
      const Event &e = t.impl()->event();
      if (e.impl()->order == 0 && !e.impl()->is_owed()) continue;  // never recorded
      if (t.impl()->priority() >= Priority::kNumPriority) {
        // handed in from outside, stamped on whatever stream the caller was on: its own wait
        if (!e.query()) e.block();
        continue;
      }
      if (e.impl()->stream == here) continue;  // stream order
      int k = 0;
      while (k < n_latest && latest[k]->impl()->stream != e.impl()->stream) ++k;
      if (k == n_latest) {
        if (n_latest == kMostStreams) {  // more streams than slots (many schedulers): wait at once
          wait_for(lane, e);
          continue;
        }
        latest[n_latest++] = &e;
      } else if (!latest[k]->impl()->is_owed() &&
                 (e.impl()->is_owed() || e.impl()->order > latest[k]->impl()->order)) {
        latest[k] = &e;  // an event still owed will be recorded at its stream's tail: it covers the others
      }
    }
    for (int k = 0; k < n_latest; ++k) wait_for(lane, *latest[k]);
    {
      // the task's name as a range in marker traces (rocprofv3 --marker-trace)
      const TraceRange range{task.impl()->name()};
      task();
    }
    // side-lane tasks get an event of their own; main-lane tasks share one that is recorded when
    // it is first needed (Event::Impl::defer), and the lane starts another after that
    const Event stamp = lane == Priority::kMain ? shared_stamp() : recorded_stamp();
    for (const auto &t : task.impl()->output()) {
      t.impl()->priority() = lane;
      replace(t.impl()->event(), stamp);
    }
    for (const auto &done : task.impl()->completed()) {
      done->priority() = lane;
      replace(done->event(), stamp);
    }
    task.impl()->completed().clear();
    return stamp;
  }
  Event shared_stamp() {
    if (!open_.impl()->is_owed()) {
      replace(open_, Event{});
      open_.impl()->defer(streams_[Priority::kMain]);
    }
    return open_;
  }
  static Event recorded_stamp() {
    Event stamp;
    stamp.record();
    return stamp;
  }
  // one more main task has arrived: side-stream work that is old enough is waited for, unless
  // it has finished already (a wait costs the main stream about 7 us even then)
  void age(std::deque<Parked> &queue) {
    for (auto &p : queue) --p.countdown;
    while (!queue.empty() && queue.back().countdown <= 0) {
      wait_for(Priority::kMain, queue.back().done);
      queue.pop_back();
    }
  }
  // The current stream (the one of `lane`) is made to wait for `e` - unless it already waits for
  // that event or for a later one recorded on the same stream, which covers it: a stream finishes
  // its events in the order it recorded them.  A training step's 25 LayerNorm forwards each read
  // parameters that the optimizer task of the assist lane wrote; one wait serves them all, where
  // each used to put a wait packet into the main stream (7-18 us of host time apiece while the
  // optimizer kernel was still running).
  void wait_for(const Priority lane, const Event &e) {
    e.impl()->settle();  // an owed record is made now; its position in the stream is known after that
    const uint64_t order = e.impl()->order;
    if (order == 0) return;  // never recorded
    auto &seen = waited_[lane];
    size_t k = 0;
    while (k < seen.size() && seen[k].stream != e.impl()->stream) ++k;
    if (k == seen.size()) seen.push_back({e.impl()->stream, 0});
    if (order <= seen[k].order) return;  // covered by an earlier wait
    if (!e.query()) e.block();
    seen[k].order = order;
  }
  static std::vector<at::Tensor> touched(const Task::Impl &body) {
    std::vector<at::Tensor> keep;
    keep.reserve(body.input().size() + body.output().size() + body.intermediate().size());
    for (const auto &t : body.input()) keep.push_back(t.impl()->tensor());
    for (const auto &t : body.output()) keep.push_back(t.impl()->tensor());
    for (const auto &t : body.intermediate()) keep.push_back(t);
    return keep;
  }

  std::recursive_mutex submit_mutex_;  // recursive: a body may submit a task of its own
  std::vector<Stream> streams_;
  // per waiting lane and recording stream: position (Event::Impl::order) of the latest event that
  // the waiting lane's stream has been made to wait for, or has seen completed
  struct Waited {
    c10::StreamId stream;
    uint64_t order;
  };
  std::vector<Waited> waited_[Priority::kNumPriority];
  Event main_done_;
  Event open_;  // the event that main-lane tasks share until somebody needs it
  std::deque<Parked> assist_, comm_;
};
}  // namespace

DynamicScheduler::DynamicScheduler(int localRank) {
  impl_ = std::make_shared<ThreeStreamScheduler>(localRank);
}
}  // namespace cs

namespace at {
bool allclose(const cs::ReadOnlyTensor &t1, const at::Tensor &t2, const double rtol, const double atol,
              const bool equal_nan) {
  t1.wait();
  return at::allclose(t1.impl()->tensor(), t2, rtol, atol, equal_nan);
}
bool allclose(const cs::ReadOnlyTensor &t1, const cs::ReadOnlyTensor &t2, const double rtol,
              const double atol, const bool equal_nan) {
  t1.wait();
  t2.wait();
  return at::allclose(t1.impl()->tensor(), t2.impl()->tensor(), rtol, atol, equal_nan);
}
bool allclose(const at::Tensor &t1, const cs::ReadOnlyTensor &t2, const double rtol, const double atol,
              const bool equal_nan) {
  t2.wait();
  return at::allclose(t1, t2.impl()->tensor(), rtol, atol, equal_nan);
}
}  // namespace at
