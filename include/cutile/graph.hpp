// Graph capture and replay on hipGraph.
//
// Mirrors cuda-async/src/cuda_graph.rs: capture (:61-137, including the
// (op result, end-capture result) failure matrix), take_output (:143-145),
// update (:161-164), launch as a DeviceOp (:179-209), scope with record()
// (:343-505), destruction order exec-then-graph (:229-244).
//
// All device pointers are baked in at capture time: to vary inputs, copy new data
// into a pre-allocated buffer with update(memcpy(...)) before each launch.  Ops
// that allocate are not graph nodes; Scope::record rejects them at compile time.
#pragma once
#include "device_op.hpp"

namespace cutile {

class GraphLaunch : public DeviceOp<GraphLaunch, Unit> {
 public:
  explicit GraphLaunch(cutile_graph_exec_t exec) : exec_(exec) {}
  Result<Unit> execute(const ExecutionContext& ctx) && { return check(cutile_graph_launch(exec_, ctx.stream()->raw())); }

 private:
  cutile_graph_exec_t exec_;
};

class Scope;

template <class T>
class HipGraph {
 public:
  HipGraph(HipGraph&& o) noexcept
      : stream_(std::move(o.stream_)), graph_(o.graph_), exec_(o.exec_), output_(std::move(o.output_)) {
    o.graph_ = nullptr;
    o.exec_ = nullptr;
  }
  HipGraph& operator=(HipGraph&&) = delete;
  HipGraph(const HipGraph&) = delete;
  ~HipGraph() {
    if (stream_) (void)stream_->device()->bind_to_thread();
    if (exec_) cutile_graph_exec_destroy(exec_);
    if (graph_) cutile_graph_destroy(graph_);
  }

  // capture: begin (relaxed) -> execute the op on the capture stream -> end ->
  // instantiate -> upload -> synchronise.  End-capture always runs.
  template <class Op>
  static Result<HipGraph<T>> capture(std::shared_ptr<Stream> stream, Op op) {
    CUTILE_TRY(stream->device()->bind_to_thread());
    CUTILE_TRY_STATUS(cutile_stream_begin_capture(stream->raw()));
    ExecutionContext ctx(stream);
    Result<T> op_result = std::move(op).execute(ctx);
    cutile_graph_t graph = nullptr;
    cutile_status_t end = cutile_stream_end_capture(stream->raw(), &graph);
    DeviceError end_err = end == CUTILE_SUCCESS ? DeviceError{} : DeviceError::from_status(end);
    if (op_result.is_err()) {
      if (end == CUTILE_SUCCESS && graph) cutile_graph_destroy(graph);
      return op_result.error();
    }
    if (end != CUTILE_SUCCESS) return end_err;
    if (!graph) return DeviceError::internal("hipStreamEndCapture returned null graph");
    return finish(std::move(stream), graph, std::move(op_result).unwrap());
  }

  // scope: record nodes one by one with plain borrows; see Scope below.
  template <class F>
  static Result<HipGraph<Unit>> scope(const std::shared_ptr<Stream>& stream, F body);

  std::optional<T> take_output() {
    auto o = std::move(output_);
    output_.reset();
    return o;
  }
  // update: run an op on the graph's stream without synchronising (e.g. memcpy of a new input).
  template <class Op>
  Result<typename Op::Output> update(Op op) const {
    ExecutionContext ctx(stream_);
    return std::move(op).execute(ctx);
  }
  GraphLaunch launch() const { return GraphLaunch(exec_); }
  const std::shared_ptr<Stream>& stream() const { return stream_; }

 private:
  friend class Scope;
  template <class U>
  friend class HipGraph;
  HipGraph(std::shared_ptr<Stream> s, cutile_graph_t g, cutile_graph_exec_t e, T out)
      : stream_(std::move(s)), graph_(g), exec_(e), output_(std::move(out)) {}
  static Result<HipGraph<T>> finish(std::shared_ptr<Stream> stream, cutile_graph_t graph, T out) {
    cutile_graph_exec_t exec = nullptr;
    cutile_status_t s = cutile_graph_instantiate(graph, &exec);
    if (s != CUTILE_SUCCESS) {
      DeviceError e = DeviceError::from_status(s);
      cutile_graph_destroy(graph);
      return e;
    }
    s = cutile_graph_upload(exec, stream->raw());
    if (s != CUTILE_SUCCESS) {
      DeviceError e = DeviceError::from_status(s);
      cutile_graph_exec_destroy(exec);
      cutile_graph_destroy(graph);
      return e;
    }
    auto synced = stream->synchronize();
    if (synced.is_err()) {
      cutile_graph_exec_destroy(exec);
      cutile_graph_destroy(graph);
      return synced.error();
    }
    return HipGraph<T>(std::move(stream), graph, exec, std::move(out));
  }
  std::shared_ptr<Stream> stream_;
  cutile_graph_t graph_ = nullptr;
  cutile_graph_exec_t exec_ = nullptr;
  std::optional<T> output_;
};

// The recording handle passed to the body of HipGraph::scope (cuda_graph.rs:343-371).
class Scope {
 public:
  // Records one node.  Only graph-node ops are accepted: kernel launches, memcpy
  // between existing buffers, plain values — nothing that allocates.
  template <class Op>
  Result<typename Op::Output> record(Op op) {
    static_assert(is_graph_node_v<Op>, "only kernel launches, memcpy and values can be recorded into a graph");
    return std::move(op).execute(ctx_);
  }

 private:
  template <class U>
  friend class HipGraph;
  explicit Scope(const std::shared_ptr<Stream>& s) : ctx_(s) {}
  ExecutionContext ctx_;
};

template <class T>
template <class F>
Result<HipGraph<Unit>> HipGraph<T>::scope(const std::shared_ptr<Stream>& stream, F body) {
  // The execution lock is held for the whole body; whatever the body does —
  // including throwing — capture is ended before this returns (cuda_graph.rs:400-505).
  CUTILE_TRY(ExecutionLock::acquire());
  auto bound = stream->device()->bind_to_thread();
  if (bound.is_err()) {
    ExecutionLock::release();
    return bound.error();
  }
  cutile_status_t begun = cutile_stream_begin_capture(stream->raw());
  if (begun != CUTILE_SUCCESS) {
    ExecutionLock::release();
    return DeviceError::from_status(begun);
  }
  Scope s(stream);
  Result<Unit> body_result = Unit{};
  std::exception_ptr thrown;
  try {
    body_result = body(s);
  } catch (...) {
    thrown = std::current_exception();
  }
  cutile_graph_t graph = nullptr;
  cutile_status_t end = cutile_stream_end_capture(stream->raw(), &graph);
  DeviceError end_err = end == CUTILE_SUCCESS ? DeviceError{} : DeviceError::from_status(end);
  ExecutionLock::release();
  if (thrown || body_result.is_err()) {
    if (end == CUTILE_SUCCESS && graph) cutile_graph_destroy(graph);
    if (thrown) std::rethrow_exception(thrown);
    return body_result.error();
  }
  if (end != CUTILE_SUCCESS) return end_err;
  if (!graph) return DeviceError::internal("hipStreamEndCapture returned null graph");
  return HipGraph<Unit>::finish(stream, graph, Unit{});
}

template <class D, class O>
Result<HipGraph<O>> DeviceOp<D, O>::graph_on(std::shared_ptr<Stream> stream) && {
  return HipGraph<O>::capture(std::move(stream), self());
}
template <class D, class O>
Result<HipGraph<O>> DeviceOp<D, O>::graph() && {
  auto stream = next_stream();
  if (stream.is_err()) return stream.error();
  return std::move(*this).graph_on(stream.value());
}

inline auto graph_scope = [](const std::shared_ptr<Stream>& stream, auto body) {
  return HipGraph<Unit>::scope(stream, std::move(body));
};

}  // namespace cutile
