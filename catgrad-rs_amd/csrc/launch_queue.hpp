// launch_queue.hpp — kernel launches handed to a second host thread.
//
// A decode step is a few thousand evaluator calls that record a graph and ~80 kernel launches that
// run it.  A launch costs the calling thread 2.5 us inside the HIP runtime: a fifth of a millisecond
// per step that the evaluator thread spends waiting on nothing it needs.  With a queue, a launch is
// a copy of the kernel's arguments into a ring slot (a tenth of a microsecond); one worker thread
// per backend takes the slots in order and makes the runtime calls.  The stream still receives
// every launch in program order, so the rule that lets storage be recycled at once - every
// consumer was enqueued on the backend's only stream before the storage is reused - holds
// unchanged.  Anything else that touches the stream (copies, events, synchronisation, frees) first
// waits for the queue to drain.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <mutex>
#include <new>
#include <thread>
#include <tuple>
#include <type_traits>
#include <utility>

namespace cgk {

class LaunchQueue {
 public:
  enum : size_t { SLOTS = 256, SLOT_BYTES = 2048 };

  explicit LaunchQueue(int device) : device_(device), slots_(new Slot[SLOTS]) {
    worker_ = std::thread([this] { run(); });
  }
  ~LaunchQueue() {
    drain();
    stop_.store(true, std::memory_order_release);
    wake();
    worker_.join();
    delete[] slots_;
  }
  LaunchQueue(const LaunchQueue &) = delete;
  LaunchQueue &operator=(const LaunchQueue &) = delete;

  // Copies a launch into the ring (waits while the ring is full).
  template <typename... KArgs, typename... Args>
  void launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t smem, hipStream_t stream, Args &&...args) {
    struct Payload {
      void (*kernel)(KArgs...);
      dim3 grid, block;
      size_t smem;
      hipStream_t stream;
      std::tuple<std::decay_t<KArgs>...> a;
    };
    static_assert(sizeof(Payload) <= SLOT_BYTES, "kernel arguments larger than a ring slot");
    static_assert(std::is_trivially_destructible<Payload>::value, "kernel arguments are plain data");
    const uint64_t h = head_.load(std::memory_order_relaxed);
    while (h - tail_.load(std::memory_order_acquire) >= SLOTS) pause();
    Slot &s = slots_[h % SLOTS];
    new (s.buf) Payload{kernel, grid, block, smem, stream, std::tuple<std::decay_t<KArgs>...>(std::forward<Args>(args)...)};
    s.run = [](void *p) {
      Payload *q = static_cast<Payload *>(p);
      std::apply(
          [q](auto &...a) { hipExtLaunchKernelGGL(q->kernel, q->grid, q->block, q->smem, q->stream, nullptr, nullptr, 0, a...); },
          q->a);
    };
    // sequentially consistent on both sides: either this thread sees the worker asleep, or the worker's
    // last look at the ring before it sleeps sees this slot
    head_.store(h + 1);
    if (sleeping_.load()) wake();
  }

  // Returns once every launch handed over so far has been given to the runtime.
  void drain() const {
    const uint64_t h = head_.load(std::memory_order_acquire);
    while (tail_.load(std::memory_order_acquire) < h) pause();
  }

  // First error a launch reported since the last call (hipSuccess if none).
  hipError_t take_error() { return (hipError_t)error_.exchange((int)hipSuccess, std::memory_order_acq_rel); }

 private:
  struct Slot {
    void (*run)(void *);
    alignas(16) unsigned char buf[SLOT_BYTES];
  };
  static void pause() {
#if defined(__x86_64__)
    __builtin_ia32_pause();
#else
    std::this_thread::yield();
#endif
  }
  void wake() {
    std::lock_guard<std::mutex> lk(m_);
    cv_.notify_one();
  }
  void run() {
    (void)hipSetDevice(device_);
    uint32_t idle = 0;
    for (;;) {
      const uint64_t t = tail_.load(std::memory_order_relaxed);
      if (head_.load(std::memory_order_acquire) == t) {
        if (stop_.load(std::memory_order_acquire)) return;
        if (++idle < 20000) {  // a few hundred microseconds of polling, then sleep until woken
          pause();
          continue;
        }
        std::unique_lock<std::mutex> lk(m_);
        sleeping_.store(true);
        cv_.wait_for(lk, std::chrono::milliseconds(50), [this, t] { return head_.load() != t || stop_.load(); });
        sleeping_.store(false);
        idle = 0;
        continue;
      }
      idle = 0;
      Slot &s = slots_[t % SLOTS];
      s.run(s.buf);
      const hipError_t e = hipGetLastError();
      if (e != hipSuccess) {
        int none = (int)hipSuccess;
        error_.compare_exchange_strong(none, (int)e, std::memory_order_acq_rel);
      }
      tail_.store(t + 1, std::memory_order_release);
    }
  }

  int device_;
  Slot *slots_;
  std::atomic<uint64_t> head_{0}, tail_{0};
  std::atomic<bool> stop_{false}, sleeping_{false};
  std::atomic<int> error_{(int)hipSuccess};
  std::mutex m_;
  std::condition_variable cv_;
  std::thread worker_;
};

}  // namespace cgk
