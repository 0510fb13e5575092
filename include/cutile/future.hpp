// DeviceFuture: a DeviceOp scheduled on a stream, polled to completion.
//
// Mirrors cuda-async/src/device_future.rs:19-33 (states), :59-154 (construction,
// completion registration), :190-323 (poll).  C++17 has no task context, so the
// waker is a plain callable: poll(waker) returns the result when ready and
// otherwise keeps `waker` to be called — from the reactor's scanner thread or a
// host callback — once the submitted work has completed.
#pragma once
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <functional>
#include <mutex>

#include "device_op.hpp"

namespace cutile {

enum class DeviceFutureState { Failed, Idle, Executing, Complete };

// Shared between a future and the completion signal (device_future.rs:35-57).
struct StreamCallbackState {
  std::atomic<bool> complete{false};
  std::mutex mu;
  std::function<void()> waker;
  void register_waker(std::function<void()> w) {
    std::lock_guard<std::mutex> lock(mu);
    waker = std::move(w);
  }
  void signal() {
    complete.store(true, std::memory_order_release);
    std::function<void()> w;
    {
      std::lock_guard<std::mutex> lock(mu);
      w = waker;
    }
    if (w) w();
  }
};

// Microseconds the first poll spins on the completion flag before it reports
// "pending" and the caller parks (device_future.rs:233-262);
// CUTILE_ASYNC_SPIN_BUDGET_US=0 sends every future through the parked path.
inline uint64_t inline_spin_budget_us() {
  static const uint64_t budget = [] {
    const char* v = std::getenv("CUTILE_ASYNC_SPIN_BUDGET_US");
    return v ? std::strtoull(v, nullptr, 10) : 20ull;
  }();
  return budget;
}

template <class Op>
class DeviceFuture {
 public:
  using T = typename Op::Output;
  DeviceFuture() = default;
  // scheduled(op, ctx) — device_future.rs:76-86
  DeviceFuture(Op op, ExecutionContext ctx) : op_(std::move(op)), ctx_(std::move(ctx)) {}
  // failed(error) — device_future.rs:88-97: the first poll yields the error.
  static DeviceFuture failed(DeviceError e) {
    DeviceFuture f;
    f.state_ = DeviceFutureState::Failed;
    f.error_ = std::move(e);
    return f;
  }
  DeviceFuture(DeviceFuture&&) = default;
  DeviceFuture& operator=(DeviceFuture&&) = default;

  DeviceFutureState state() const { return state_; }

  // One poll.  Empty = pending (the waker will be called); otherwise the result.
  std::optional<Result<T>> poll(std::function<void()> waker) {
    if (state_ == DeviceFutureState::Failed) {
      state_ = DeviceFutureState::Complete;
      return Result<T>(std::move(*error_));
    }
    if (!cb_) cb_ = std::make_shared<StreamCallbackState>();
    switch (state_) {
      case DeviceFutureState::Idle: {
        auto locked = ExecutionLock::acquire();
        if (locked.is_err()) {
          state_ = DeviceFutureState::Complete;
          return Result<T>(locked.error());
        }
        cb_->register_waker(std::move(waker));
        if (!op_ || !ctx_) {
          ExecutionLock::release();
          state_ = DeviceFutureState::Complete;
          return Result<T>(DeviceError::internal("Cannot execute future without setting stream on which to execute."));
        }
        Op op = std::move(*op_);
        op_.reset();
        auto r = std::move(op).execute(*ctx_);
        if (r.is_err()) {
          ExecutionLock::release();
          state_ = DeviceFutureState::Complete;
          return Result<T>(r.error());
        }
        result_.emplace(std::move(r).unwrap());
        // Register the completion signal, once.  The callback owns a reference
        // to the shared state, so it may fire after this future is gone.
        auto* held = new std::shared_ptr<StreamCallbackState>(cb_);
        cutile_status_t s = cutile_completion_register(ctx_->stream()->raw(), &DeviceFuture::on_complete, held);
        ExecutionLock::release();
        if (s != CUTILE_SUCCESS) {
          delete held;
          state_ = DeviceFutureState::Complete;
          return Result<T>(DeviceError::from_status(s));
        }
        state_ = DeviceFutureState::Executing;
        // Inline fast path (device_future.rs:233-262 spins on the stream before registering): here the
        // registration comes first, it is one 32-bit stream write into pinned memory, and the bounded spin
        // watches the completion flag it leads to.  A hipStreamQuery poll loop reported the completion of one small
        // kernel about 10 us later than this flag (22.6 against 13.0 us from launch), past the default budget, so
        // short operations always fell through to the parked path.
        if (uint64_t budget = inline_spin_budget_us()) {
          auto deadline = std::chrono::steady_clock::now() + std::chrono::microseconds(budget);
          while (!cb_->complete.load(std::memory_order_acquire) && std::chrono::steady_clock::now() < deadline) {}
          if (cb_->complete.load(std::memory_order_acquire)) {
            state_ = DeviceFutureState::Complete;
            return Result<T>(std::move(*result_));
          }
        }
        return std::nullopt;
      }
      case DeviceFutureState::Executing: {
        if (cb_->complete.load(std::memory_order_acquire)) {
          state_ = DeviceFutureState::Complete;
          return Result<T>(std::move(*result_));
        }
        cb_->register_waker(std::move(waker));
        // The signal may have fired between the check and the re-registration.
        if (cb_->complete.load(std::memory_order_acquire)) {
          state_ = DeviceFutureState::Complete;
          return Result<T>(std::move(*result_));
        }
        return std::nullopt;
      }
      case DeviceFutureState::Complete:
      default:
        throw std::logic_error("Poll called after completion.");
    }
  }

  // Drives the future on the calling thread: poll, sleep until woken, poll again.
  Result<T> block_on() {
    struct Parker {
      std::mutex mu;
      std::condition_variable cv;
      bool woken = false;
    };
    auto parker = std::make_shared<Parker>();
    for (;;) {
      auto r = poll([parker] {
        {
          std::lock_guard<std::mutex> lock(parker->mu);
          parker->woken = true;
        }
        parker->cv.notify_one();
      });
      if (r) return std::move(*r);
      std::unique_lock<std::mutex> lock(parker->mu);
      parker->cv.wait(lock, [&] { return parker->woken; });
      parker->woken = false;
    }
  }

 private:
  static void on_complete(void* p) {
    auto* held = static_cast<std::shared_ptr<StreamCallbackState>*>(p);
    (*held)->signal();
    delete held;
  }
  std::optional<Op> op_;
  std::optional<ExecutionContext> ctx_;
  std::optional<T> result_;
  std::optional<DeviceError> error_;
  DeviceFutureState state_ = DeviceFutureState::Idle;
  std::shared_ptr<StreamCallbackState> cb_;
};

template <class D, class O>
DeviceFuture<D> DeviceOp<D, O>::schedule_on(const std::shared_ptr<Stream>& stream) && {
  return DeviceFuture<D>(self(), ExecutionContext(stream));
}
template <class D, class O>
DeviceFuture<D> DeviceOp<D, O>::into_future() && {
  // A scheduling failure becomes a failed future, not an exception (cutile-macro/src/_module.rs:924-934).
  auto stream = next_stream();
  if (stream.is_err()) return DeviceFuture<D>::failed(stream.error());
  return std::move(*this).schedule_on(stream.value());
}
template <class D, class O>
Result<O> DeviceOp<D, O>::wait() && {
  return std::move(*this).into_future().block_on();
}

}  // namespace cutile
