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
  void block() { event.block(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA()); }
  void record() {
    static std::atomic<uint64_t> counter{0};
    order = ++counter;
    event.record();
  }
  // position of the last record() among all records of the process; 0 = never recorded.
  // Two events recorded on one stream complete in this order.
  uint64_t order = 0;
  [[nodiscard]] bool query() const { return event.query(); }
  void synchronize() const { event.synchronize(); }

 private:
  // Events here order streams of one device and tell the host that work has finished; the data
  // itself reaches the host through stream-ordered copies.  hipEventReleaseToDevice is the
  // runtime's flag for exactly that: a record releases at device scope, so the stream waits,
  // queries and host synchronisations that the scheduler builds on these events synchronize
  // with the recorded work for every reader on this device, without the write-back to system
  // scope of a default event (which costs the recording stream ~2.7 us here instead of ~0.9 us).
  at::cuda::CUDAEvent event{hipEventDisableTiming | hipEventReleaseToDevice};
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
    main_done_.block();
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
  static Event run(const Task &task, const Priority lane) {
    // of the inputs that another lane produced, the one stamped last per lane is waited for:
    // a stream finishes its events in the order it recorded them, so that wait covers the rest
    // (each wait is a packet that stalls this stream for microseconds even when it is granted)
    // tensors whose last launches were put off get them now, before the body reads or rewrites them
    for (const auto &t : task.impl()->input()) t.impl()->settle();
    for (const auto &t : task.impl()->output()) t.impl()->settle();
    const Event *latest[Priority::kNumPriority] = {};
    for (const auto &t : task.impl()->input()) {
      const Priority from = t.impl()->priority();
      if (from == lane) continue;
      const Event &e = t.impl()->event();
      if (from >= Priority::kNumPriority) {
        // handed in from outside, stamped on whatever stream the caller was on: its own wait
        if (!e.query()) e.block();
      } else if (latest[from] == nullptr || e.impl()->order > latest[from]->impl()->order) {
        latest[from] = &e;
      }
    }
    for (const Event *e : latest) {
      if (e != nullptr && !e->query()) e->block();
    }
    {
      // the task's name as a range in marker traces (rocprofv3 --marker-trace)
      const TraceRange range{task.impl()->name()};
      task();
    }
    Event stamp;
    stamp.record();
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
  // one more main task has arrived: side-stream work that is old enough is waited for, unless
  // it has finished already (a wait costs the main stream about 7 us even then)
  static void age(std::deque<Parked> &queue) {
    for (auto &p : queue) --p.countdown;
    while (!queue.empty() && queue.back().countdown <= 0) {
      if (!queue.back().done.query()) queue.back().done.block();
      queue.pop_back();
    }
  }
  static std::vector<at::Tensor> touched(const Task::Impl &body) {
    std::vector<at::Tensor> keep;
    keep.reserve(body.input().size() + body.output().size() + body.intermediate().size());
    for (const auto &t : body.input()) keep.push_back(t.impl()->tensor());
    for (const auto &t : body.output()) keep.push_back(t.impl()->tensor());
    for (const auto &t : body.intermediate()) keep.push_back(t);
    return keep;
  }

  std::vector<Stream> streams_;
  Event main_done_;
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
