// DeviceOp: a lazy description of GPU work, and its combinators.
//
// Mirrors cuda-async/src/device_operation.rs:185-385 (trait + execution
// methods), :615-1481 (Value, AndThen, Zip, Select/unzip, SharedDeviceOp,
// BoxedDeviceOp).  An op is a move-only value; execute() consumes it
// (rvalue-qualified) and enqueues its work on the context's stream without
// waiting.  Only sync()/sync_on()/wait() make the result safe to read.
//
// A type is a DeviceOp when it derives from DeviceOp<Derived, Output> and has
//     Result<Output> execute(const ExecutionContext&) &&;
#pragma once
#include <atomic>
#include <functional>
#include <memory>
#include <mutex>
#include <tuple>
#include <type_traits>
#include <utility>

#include "runtime.hpp"

namespace cutile {

// ---- thread-local execution lock (device_operation.rs:27-55) -------------------------------
struct ExecutionLock {
  static Result<Unit> acquire() { return check(cutile_execution_lock_acquire()); }
  static void release() { cutile_execution_lock_release(); }
};

struct DeviceOpTag {};
template <class T>
inline constexpr bool is_device_op_v = std::is_base_of_v<DeviceOpTag, std::decay_t<T>>;

// Marker for operations that may be recorded into a graph: they neither allocate
// nor free device memory (device_operation.rs:389-406).
template <class Op, class = void>
struct is_graph_node : std::false_type {};
template <class Op>
inline constexpr bool is_graph_node_v = is_graph_node<std::decay_t<Op>>::value;

template <class T>
class Value;
template <class Op, class F>
class AndThen;
template <class T>
class BoxedDeviceOp;
template <class T>
class SharedDeviceOp;
template <class Op>
class DeviceFuture;
template <class T>
class HipGraph;
template <size_t I, class Op>
class Select;

template <class T>
Value<std::decay_t<T>> value(T&& v);

template <class Derived, class Out>
class DeviceOp : public DeviceOpTag {
 public:
  using Output = Out;
  Derived&& self() { return static_cast<Derived&&>(*this); }

  // then: follow-up GPU work on the same stream (device_operation.rs:214-224).
  template <class F>
  auto then(F f) && {
    return AndThen<Derived, F>(self(), std::move(f));
  }
  // map: transform the output, no GPU work (device_operation.rs:238-252).
  template <class F>
  auto map(F f) && {
    return std::move(*this).then([f = std::move(f)](Out x) mutable { return value(f(std::move(x))); });
  }
  // inspect: peek at the output and pass it on (device_operation.rs:253-272).
  template <class F>
  auto inspect(F f) && {
    return std::move(*this).map([f = std::move(f)](Out x) mutable {
      f(static_cast<const Out&>(x));
      return x;
    });
  }
  // first / last of a tuple output.
  auto first() && {
    return std::move(*this).map([](Out t) { return std::get<0>(std::move(t)); });
  }
  auto last() && {
    return std::move(*this).map([](Out t) { return std::get<std::tuple_size_v<Out> - 1>(std::move(t)); });
  }
  // unzip: one op per tuple element; the source runs once (device_operation.rs:971-1011).
  auto unzip() &&;
  BoxedDeviceOp<Out> boxed() &&;
  // shared: cloneable, execute-once, output becomes shared_ptr<Out> (device_operation.rs:447-493).
  SharedDeviceOp<Out> shared() &&;

  // async_on: enqueue on `stream` and return at once; the output may still be
  // in flight on the device (the reference marks this unsafe, device_operation.rs:364-370).
  Result<Out> async_on(const std::shared_ptr<Stream>& stream) && {
    ExecutionContext ctx(stream);
    return self().execute(ctx);
  }
  // sync_on: take the execution lock, execute, synchronise the stream, release (device_operation.rs:376-384).
  Result<Out> sync_on(const std::shared_ptr<Stream>& stream) && {
    CUTILE_TRY(ExecutionLock::acquire());
    ExecutionContext ctx(stream);
    Result<Out> res = self().execute(ctx);
    Result<Unit> synced = stream->synchronize();
    ExecutionLock::release();
    if (synced.is_err()) return synced.error();
    return res;
  }
  // sync: stream from the thread's default policy (device_operation.rs:353-356).
  Result<Out> sync() && {
    auto stream = next_stream();
    if (stream.is_err()) return stream.error();
    return std::move(*this).sync_on(stream.value());
  }
  // schedule / into_future: a future on a policy-chosen stream (device_operation.rs:203-213).
  DeviceFuture<Derived> into_future() &&;
  DeviceFuture<Derived> schedule_on(const std::shared_ptr<Stream>& stream) &&;
  // wait: what `.await` does, driven to completion on the calling thread.
  Result<Out> wait() &&;
  // graph_on / graph: capture into a replayable graph (device_operation.rs:338-352).
  Result<HipGraph<Out>> graph_on(std::shared_ptr<Stream> stream) &&;
  Result<HipGraph<Out>> graph() &&;
};

// ---- Value (device_operation.rs:684-722) ---------------------------------------------------
template <class T>
class Value : public DeviceOp<Value<T>, T> {
 public:
  explicit Value(T v) : v_(std::move(v)) {}
  Result<T> execute(const ExecutionContext&) && { return std::move(v_); }

 private:
  T v_;
};
template <class T>
Value<std::decay_t<T>> value(T&& v) {
  return Value<std::decay_t<T>>(std::forward<T>(v));
}
template <class T>
struct is_graph_node<Value<T>> : std::true_type {};

// IntoDeviceOp: launchers take ops and plain values alike (device_operation.rs:615-680).
template <class X>
auto into_op(X&& x) {
  if constexpr (is_device_op_v<X>)
    return std::decay_t<X>(std::forward<X>(x));
  else
    return value(std::forward<X>(x));
}
template <class X>
using into_op_t = decltype(into_op(std::declval<X>()));

// ---- AndThen -------------------------------------------------------------------------------
template <class Op, class F>
class AndThen : public DeviceOp<AndThen<Op, F>, typename std::invoke_result_t<F, typename Op::Output>::Output> {
 public:
  using Next = std::invoke_result_t<F, typename Op::Output>;
  static_assert(is_device_op_v<Next>, "the closure given to then() must return a DeviceOp");
  AndThen(Op&& op, F f) : op_(std::move(op)), f_(std::move(f)) {}
  Result<typename Next::Output> execute(const ExecutionContext& ctx) && {
    auto first = std::move(op_).execute(ctx);
    if (first.is_err()) return first.error();
    return f_(std::move(first).unwrap()).execute(ctx);
  }

 private:
  Op op_;
  F f_;
};

// ---- Zip (device_operation.rs:775-970) -----------------------------------------------------
template <class... Ops>
class Zip : public DeviceOp<Zip<Ops...>, std::tuple<typename Ops::Output...>> {
 public:
  using Out = std::tuple<typename Ops::Output...>;
  explicit Zip(Ops&&... ops) : ops_(std::move(ops)...) {}
  Result<Out> execute(const ExecutionContext& ctx) && {
    return run(ctx, std::index_sequence_for<Ops...>{});
  }

 private:
  template <size_t... I>
  Result<Out> run(const ExecutionContext& ctx, std::index_sequence<I...>) {
    // Elements execute in argument order on the same stream.
    std::tuple<std::optional<typename Ops::Output>...> parts;
    std::optional<DeviceError> err;
    (void)std::initializer_list<int>{(run_one<I>(ctx, parts, err), 0)...};
    if (err) return *err;
    return Out(std::move(*std::get<I>(parts))...);
  }
  template <size_t I, class Parts>
  void run_one(const ExecutionContext& ctx, Parts& parts, std::optional<DeviceError>& err) {
    if (err) return;
    auto r = std::move(std::get<I>(ops_)).execute(ctx);
    if (r.is_err())
      err = r.error();
    else
      std::get<I>(parts).emplace(std::move(r).unwrap());
  }
  std::tuple<Ops...> ops_;
};
template <class... Xs>
auto zip(Xs&&... xs) {
  return Zip<into_op_t<Xs>...>(into_op(std::forward<Xs>(xs))...);
}
template <class... Ops>
struct is_graph_node<Zip<Ops...>> : std::bool_constant<(is_graph_node_v<Ops> && ...)> {};
template <class Op, class F>
struct is_graph_node<AndThen<Op, F>> : std::false_type {};

// ---- Boxed (type erasure) ------------------------------------------------------------------
template <class T>
class BoxedDeviceOp : public DeviceOp<BoxedDeviceOp<T>, T> {
 public:
  template <class Op>
  explicit BoxedDeviceOp(Op&& op) : inner_(std::make_unique<Model<std::decay_t<Op>>>(std::move(op))) {}
  Result<T> execute(const ExecutionContext& ctx) && {
    if (!inner_) return DeviceError::internal("boxed DeviceOp was already executed");
    auto p = std::move(inner_);
    return p->run(ctx);
  }

 private:
  struct Concept {
    virtual ~Concept() = default;
    virtual Result<T> run(const ExecutionContext&) = 0;
  };
  template <class Op>
  struct Model : Concept {
    explicit Model(Op&& o) : op(std::move(o)) {}
    Result<T> run(const ExecutionContext& ctx) override { return std::move(op).execute(ctx); }
    Op op;
  };
  std::unique_ptr<Concept> inner_;
};
template <class D, class O>
BoxedDeviceOp<O> DeviceOp<D, O>::boxed() && {
  return BoxedDeviceOp<O>(self());
}

// ---- Shared: clone + execute once ----------------------------------------------------------
template <class T>
class SharedDeviceOp : public DeviceOp<SharedDeviceOp<T>, std::shared_ptr<T>> {
 public:
  explicit SharedDeviceOp(BoxedDeviceOp<T> op) : st_(std::make_shared<State>()) { st_->op.emplace(std::move(op)); }
  explicit SharedDeviceOp(std::shared_ptr<T> ready) : st_(std::make_shared<State>()) { st_->result = std::move(ready); }
  SharedDeviceOp(const SharedDeviceOp&) = default;  // clones share the state
  SharedDeviceOp(SharedDeviceOp&&) = default;
  Result<std::shared_ptr<T>> execute(const ExecutionContext& ctx) && {
    std::lock_guard<std::mutex> lock(st_->mu);
    if (st_->result) return st_->result;
    if (st_->error) return *st_->error;
    auto r = std::move(*st_->op).execute(ctx);
    st_->op.reset();
    if (r.is_err()) {
      st_->error = r.error();
      return r.error();
    }
    st_->result = std::make_shared<T>(std::move(r).unwrap());
    return st_->result;
  }

 private:
  struct State {
    std::mutex mu;
    std::optional<BoxedDeviceOp<T>> op;
    std::shared_ptr<T> result;
    std::optional<DeviceError> error;
  };
  std::shared_ptr<State> st_;
};
template <class D, class O>
SharedDeviceOp<O> DeviceOp<D, O>::shared() && {
  return SharedDeviceOp<O>(std::move(*this).boxed());
}
// shared(arc): wrap an existing shared_ptr as an already computed op.
template <class T>
SharedDeviceOp<T> shared(std::shared_ptr<T> ready) {
  return SharedDeviceOp<T>(std::move(ready));
}
// unwrap_arc: owned T back from a uniquely held shared_ptr<T>; throws when shared.
template <class T>
T unwrap_arc(std::shared_ptr<T> p) {
  if (p.use_count() != 1) throw std::logic_error("unwrap_arc: the Arc has multiple owners");
  return std::move(*p);
}

// ---- Select / unzip ------------------------------------------------------------------------
template <class Tuple>
struct UnzipState {
  std::mutex mu;
  std::optional<BoxedDeviceOp<Tuple>> op;
  std::optional<Tuple> result;
  std::optional<DeviceError> error;
};
template <size_t I, class Tuple>
class SelectOp : public DeviceOp<SelectOp<I, Tuple>, std::tuple_element_t<I, Tuple>> {
 public:
  using Elem = std::tuple_element_t<I, Tuple>;
  explicit SelectOp(std::shared_ptr<UnzipState<Tuple>> st) : st_(std::move(st)) {}
  Result<Elem> execute(const ExecutionContext& ctx) && {
    std::lock_guard<std::mutex> lock(st_->mu);
    if (!st_->result && !st_->error) {
      auto r = std::move(*st_->op).execute(ctx);
      st_->op.reset();
      if (r.is_err())
        st_->error = r.error();
      else
        st_->result.emplace(std::move(r).unwrap());
    }
    if (st_->error) return *st_->error;
    return std::move(std::get<I>(*st_->result));
  }

 private:
  std::shared_ptr<UnzipState<Tuple>> st_;
};
template <class Tuple, size_t... I>
auto make_selects(std::shared_ptr<UnzipState<Tuple>> st, std::index_sequence<I...>) {
  return std::make_tuple(SelectOp<I, Tuple>(st)...);
}
template <class D, class O>
auto DeviceOp<D, O>::unzip() && {
  auto st = std::make_shared<UnzipState<O>>();
  st->op.emplace(std::move(*this).boxed());
  return make_selects<O>(st, std::make_index_sequence<std::tuple_size_v<O>>{});
}

}  // namespace cutile
