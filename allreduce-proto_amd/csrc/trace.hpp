// Host-side pipeline trace, in the reference's categories and file format.
//
// The reference compiles this in with -DUSE_TRACE: TRACE(v) pushes a CLOCK_MONOTONIC_RAW timestamp
// (ibcomm/allreduce_cuda_impl.h:18-22, ibcomm/util.h:62-70), events come in begin/end pairs in seven
// vectors (ibcomm/ibverbs_communicator.h:168-189), and the destructor writes
// ${IBCOMM_TRACE_FILE:-ibcomm_trace}_<rank>.dat with one CSV line per category,
// "name,start_ms,duration_ms,start_ms,duration_ms,..." in scientific notation relative to the timer
// base (ibcomm/ibverbs_communicator.cpp:157-216).  Here tracing is switched on at run time
// (IBCOMM_HIP_TRACE=1) and costs one branch per event when off.  What the categories mean for the
// stream-ordered engine:
//   received            a message was taken from a peer's channel
//   reduced             the reduction of a batch of chunks was enqueued and its result handed on
//   issue-send          a send was posted
//   issue-copy-kernel   a landing copy or a gather was enqueued
//   issue-redu-kernel   a reduction launch was enqueued
//   issue-recv          a pool slot was reserved for an incoming message
//   other               Begin / Finish of a collective; in a graph replay, the call that launches
//                       the graph and the wait for its completion flag
//
// Beyond the reference: when device work was traced, three more lines in the same format hold DEVICE
// durations, measured with HIP events on the streams the work ran on (without any, the file has the
// reference's seven lines and nothing else):
//   device-redu-kernel  each reduction launch (eager issue only)
//   device-copy-kernel  each landing copy and each gather (eager issue only)
//   device-graph        each replay of a recorded call, first kernel to last
// Their start times are on the host clock: the moment the first traced launch was issued plus the
// device time elapsed since that launch began.
#pragma once

#include <time.h>

#include <fstream>
#include <string>
#include <vector>

namespace ibcomm_hip {

class Trace {
 public:
  enum Category { kReceived, kReduced, kIssueSend, kIssueCopyKernel, kIssueReduKernel, kIssueRecv, kOther, kCategories };
  enum DeviceCategory { kDeviceReduce, kDeviceCopy, kDeviceGraph, kDeviceCategories };

  void Enable(bool on) { enabled_ = on; }
  bool enabled() const { return enabled_; }
  void SetTimerBase() { clock_gettime(CLOCK_MONOTONIC_RAW, &base_); has_base_ = true; }  // cpp:214-216

  void Mark(Category c) {
    if (!enabled_) return;
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC_RAW, &ts);
    if (!has_base_) { base_ = ts; has_base_ = true; }  // the reference leaves the base uninitialised unless SetTimerBase is called
    events_[c].push_back(ts);
  }

  // Takes back the last Mark of a pair that turned out not to happen (a poll that found nothing).
  void Unmark(Category c) {
    if (enabled_ && !events_[c].empty()) events_[c].pop_back();
  }

  size_t pairs(Category c) const { return events_[c].size() / 2; }

  // Milliseconds on the host clock since the timer base (sets the base if there is none yet).
  double NowMs() {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC_RAW, &ts);
    if (!has_base_) { base_ = ts; has_base_ = true; }
    return Millis(base_, ts);
  }
  void AddDevice(DeviceCategory c, double start_ms, double duration_ms) {
    if (!enabled_) return;
    device_[c].push_back(start_ms);
    device_[c].push_back(duration_ms);
  }
  size_t device_spans(DeviceCategory c) const { return device_[c].size() / 2; }
  double device_total_ms(DeviceCategory c) const {
    double t = 0;
    for (size_t i = 1; i < device_[c].size(); i += 2) t += device_[c][i];
    return t;
  }

  // DumpTrace, cpp:183-212.
  bool Dump(const std::string& path) const {
    static const char* names[kCategories] = {"received", "reduced", "issue-send", "issue-copy-kernel",
                                             "issue-redu-kernel", "issue-recv", "other"};
    std::ofstream out(path.c_str());
    if (!out.good()) return false;
    out << std::scientific;
    for (int c = 0; c < kCategories; c++) {
      out << names[c] << ",";
      const std::vector<struct timespec>& v = events_[c];
      for (size_t i = 0; i + 1 < v.size(); i += 2) out << Millis(base_, v[i]) << "," << Millis(v[i], v[i + 1]) << ",";
      out << std::endl;
    }
    // The reference's file ends here.  The device lines follow only when there is something to put
    // in them, so a consumer that expects the seven lines finds exactly those unless device work
    // was traced.
    bool any_device = false;
    for (int c = 0; c < kDeviceCategories; c++) any_device = any_device || !device_[c].empty();
    static const char* device_names[kDeviceCategories] = {"device-redu-kernel", "device-copy-kernel", "device-graph"};
    for (int c = 0; any_device && c < kDeviceCategories; c++) {
      out << device_names[c] << ",";
      for (double x : device_[c]) out << x << ",";
      out << std::endl;
    }
    return true;
  }

  void Clear() {
    for (auto& v : events_) v.clear();
    for (auto& v : device_) v.clear();
  }

 private:
  static double Millis(const struct timespec& a, const struct timespec& b) {
    return (b.tv_sec - a.tv_sec) * 1e3 + (b.tv_nsec - a.tv_nsec) * 1e-6;
  }
  bool enabled_ = false;
  bool has_base_ = false;
  struct timespec base_ = {};
  std::vector<struct timespec> events_[kCategories];
  std::vector<double> device_[kDeviceCategories];  // start_ms, duration_ms, start_ms, ...
};

// Begin/end pair around a scope.
class TraceScope {
 public:
  TraceScope(Trace* t, Trace::Category c) : t_(t), c_(c) { t_->Mark(c_); }
  ~TraceScope() { t_->Mark(c_); }

 private:
  Trace* t_;
  Trace::Category c_;
};

}  // namespace ibcomm_hip
