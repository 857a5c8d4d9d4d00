// Run-time choice between alternatives by timing them: the interface of
// flashlight/fl/common/DynamicBenchmark.h (DynamicBenchmarkOptions<T>, DynamicBenchmark::audit, the
// process-wide benchmark mode), which fl::conv2d hands to the extension's backward passes
// (flashlight/fl/autograd/Functions.cpp:1372-1388) and the cuDNN extension uses to pick a kernel
// mode (cudnn/Conv2D.cpp:467-520).  Here the alternatives are the kernel families ("plans") of
// libflhip's backward passes.
//
// One addition to the reference's interface: an options object can be told that the option just
// tried is unusable (penalise()), for plans the library declines for a geometry.
#pragma once

#include <cstddef>
#include <functional>
#include <memory>
#include <stdexcept>
#include <unordered_set>
#include <vector>

namespace fl {

// flashlight/fl/common/Defines.h:100
constexpr std::size_t kDynamicBenchmarkDefaultCount = 10;

struct DynamicBenchmarkOptionsBase {
  virtual ~DynamicBenchmarkOptionsBase() = default;
  virtual void accumulateTimeToCurrentOption(double /*time*/, bool /*incrementCount*/ = true) {
    throw std::logic_error("DynamicBenchmarkOptionsBase::accumulateTimeToCurrentOption - unimplemented");
  }
  virtual bool timingsComplete() {
    throw std::logic_error("DynamicBenchmarkOptionsBase::timingsComplete - unimplemented");
  }

 protected:
  DynamicBenchmarkOptionsBase() = default;
};

// A list of distinct options.  Every option is tried benchCount times, in list order; after
// that the option with the smallest accumulated time is the current one for good (until reset()).
template <typename T>
struct DynamicBenchmarkOptions : DynamicBenchmarkOptionsBase {
  DynamicBenchmarkOptions(std::vector<T> options, std::size_t benchCount)
      : options_(std::move(options)), benchCount_(benchCount), tally_(options_.size()) {
    if (options_.empty())
      throw std::invalid_argument("DynamicBenchmarkOptions: Options must be passed vector with at least one element");
  }
  DynamicBenchmarkOptions(const std::unordered_set<T>& options, std::size_t benchCount)
      : DynamicBenchmarkOptions(std::vector<T>(options.begin(), options.end()), benchCount) {}

  // the option to use now: the first one that still lacks timings, or the winner
  T updateState() {
    if (!complete_) {
      for (std::size_t i = 0; i < options_.size(); ++i)
        if (tally_[i].count < benchCount_) {
          current_ = i;
          return options_[i];
        }
      std::size_t best = 0;
      for (std::size_t i = 1; i < options_.size(); ++i)
        if (tally_[i].time < tally_[best].time) best = i;
      current_ = best;
      complete_ = true;
    }
    return options_[current_];
  }
  T currentOption() { return updateState(); }
  bool timingsComplete() override {
    updateState();
    return complete_;
  }
  void accumulateTimeToCurrentOption(double time, bool incrementCount = true) override {
    if (timingsComplete())
      throw std::invalid_argument(
          "Options::accumulateTimeToCurrentOption: Tried to accumulate time when benchmarking is complete");
    tally_[current_].time += time;
    if (incrementCount) ++tally_[current_].count;
  }
  // The option being tried cannot be used (the library declined it): it gets no further tries and
  // cannot win.  Not in the reference, whose options are all valid everywhere.
  void penalise() {
    if (timingsComplete()) return;
    tally_[current_].time = 1e300;
    tally_[current_].count = benchCount_;
  }
  void reset() {
    for (auto& t : tally_) t = Tally{};
    complete_ = false;
    current_ = 0;
  }
  // accumulated seconds and number of timings of option i (for reports and tests)
  double timeOf(std::size_t i) const { return tally_.at(i).time; }
  std::size_t countOf(std::size_t i) const { return tally_.at(i).count; }
  const std::vector<T>& options() const { return options_; }

 private:
  struct Tally {
    double time = 0.;
    std::size_t count = 0;
  };
  const std::vector<T> options_;
  const std::size_t benchCount_;
  std::vector<Tally> tally_;
  bool complete_ = false;
  std::size_t current_ = 0;   // the first option is the default
};

class DynamicBenchmark {
 public:
  explicit DynamicBenchmark(std::shared_ptr<DynamicBenchmarkOptionsBase> options) : options_(std::move(options)) {}
  virtual ~DynamicBenchmark() = default;

  // Runs `function`.  While benchmark mode is on and the options still lack timings, the time
  // from a device synchronisation before it to one after it goes to the current option.
  void audit(const std::function<void()>& function, bool incrementCount = true);

  template <typename T>
  std::shared_ptr<T> getOptions() const {
    return std::static_pointer_cast<T>(options_);
  }

  static void setBenchmarkMode(bool mode);
  static bool getBenchmarkMode();

 private:
  std::shared_ptr<DynamicBenchmarkOptionsBase> options_;
};

namespace detail {
// one benchmark per backward pass of a convolution; kept by the module that owns the weights
// (flashlight/fl/nn/modules/Conv2D.h:206)
struct ConvBenchmarks {
  std::shared_ptr<DynamicBenchmark> bwdFilterBenchmark;
  std::shared_ptr<DynamicBenchmark> bwdDataBenchmark;
  std::shared_ptr<DynamicBenchmark> bwdBiasBenchmark;
};
}  // namespace detail

}  // namespace fl
