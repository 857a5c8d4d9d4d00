// A hook on every device operation of the host layer: the extension's virtuals, the
// caller closures of Functions.cpp and Tensor::astype report themselves to one
// process-wide observer, if one is set.  Used to time a training step per operation
// (StepProfiler below) and, in the test programs, to replay every operation of a real
// step on the CPU checker with the operation's own device inputs.  With no observer
// set an operation pays one pointer test.
//
// Flashlight has no such hook at this boundary; its nearest tools are the
// DynamicBenchmark options of the cuDNN extension
// (flashlight/fl/autograd/tensor/backend/cudnn/CudnnAutogradExtension.h:25) and
// external profilers.
#pragma once

#include <map>
#include <string>
#include <vector>

#include "HipTensor.h"

namespace fl {
namespace detail {

// What an operation did.  Tensors are handles onto the device buffers (no copies),
// listed in the order documented at the operation; ints / reals carry its geometry.
struct OpEvent {
  const char* op = "";
  std::vector<Tensor> inputs, outputs;
  std::vector<long long> ints;
  std::vector<double> reals;
};

class OpObserver {
 public:
  virtual ~OpObserver() = default;
  // before the operation enqueues anything
  virtual void begin(const char* /*op*/) {}
  // after it has enqueued everything
  virtual void end(const OpEvent& /*event*/) {}
  // in place of end() when the operation left without reporting: it threw, or it handed its
  // work to another operation and returned.  Every begin() is followed by exactly one of the two.
  virtual void abort(const char* /*op*/) {}
};

OpObserver* opObserver();
// nullptr removes the observer; the observer is not owned
void setOpObserver(OpObserver* observer);

// Brackets one operation.  Usage:
//   OpScope scope("relu");  ... enqueue ...;  if (scope.on()) scope.done({x}, {y});
class OpScope {
 public:
  explicit OpScope(const char* op) : observer_(opObserver()), op_(op) {
    if (observer_) observer_->begin(op);
  }
  ~OpScope() {
    if (observer_ && !finished_) observer_->abort(op_);
  }
  OpScope(const OpScope&) = delete;
  OpScope& operator=(const OpScope&) = delete;
  bool on() const { return observer_ != nullptr; }
  void done(std::vector<Tensor> inputs, std::vector<Tensor> outputs, std::vector<long long> ints = {},
            std::vector<double> reals = {}) {
    OpEvent e;
    e.op = op_;
    e.inputs = std::move(inputs);
    e.outputs = std::move(outputs);
    e.ints = std::move(ints);
    e.reals = std::move(reals);
    finished_ = true;
    observer_->end(e);
  }

 private:
  OpObserver* observer_;
  const char* op_;
  bool finished_ = false;
};

}  // namespace detail

// Times every operation of the host layer with a pair of HIP events on the backend
// stream and sums by operation name.  Operations nested in another one (the casts a
// closure makes inside an extension call) count towards the outer one.  collect()
// waits for the stream; `gaps` is the part of the span between the first and the last
// operation during which no operation was running on the device (host-side latency).
class StepProfiler : public detail::OpObserver {
 public:
  struct Entry {
    double ms = 0;
    long calls = 0;
  };
  StepProfiler();
  ~StepProfiler() override;
  void begin(const char* op) override;
  void end(const detail::OpEvent& event) override;
  void abort(const char* op) override;
  // milliseconds per operation name since the last collect(), plus "(gaps)" and "(span)"
  std::map<std::string, Entry> collect();

 private:
  struct Impl;
  Impl* impl_;
};

}  // namespace fl
