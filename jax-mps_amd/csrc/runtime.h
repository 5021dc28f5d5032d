// Host runtime: device singleton with a caching allocator and one compute stream,
// device buffers, and the executor that replays a compiled plan.  Replaces the
// reference's MlxClient / MlxBuffer / MlxExecutable (src/pjrt_plugin/mlx_client.h:27-31,
// mlx_buffer.h:46-84, mlx_executable.h:41-77).
#pragma once

#include <atomic>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "hip_abi.h"
#include "plan.h"

namespace mi355 {

struct RuntimeError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

class Device {
 public:
  static Device& get();            // throws RuntimeError when no GPU is usable
  static bool available(std::string* why);

  void* alloc(size_t bytes);       // stream-ordered reuse: blocks are recycled without waiting
  void release(void* ptr);
  mi355_stream_t stream() const { return stream_; }
  const std::string& arch() const { return arch_; }
  const std::string& name() const { return name_; }
  int computeUnits() const { return cus_; }
  size_t totalMemory() const { return totalMem_; }
  void sync();

  // statistics for PJRT_Device_MemoryStats
  int64_t bytesInUse() const { return inUse_; }
  int64_t peakBytesInUse() const { return peak_; }
  int64_t numAllocs() const { return numAllocs_; }
  int64_t largestAlloc() const { return largest_; }
  int64_t bytesReserved() const { return reserved_; }

  // compiled-kernel cache shared by all executables (key: source text)
  mi355_function_t findKernel(const std::string& source);
  void storeKernel(const std::string& source, mi355_function_t fn);

  void* pinnedScratch() const { return pinned_; }   // 4 KiB pinned host buffer for predicate read-back

 private:
  Device();
  std::mutex mu_;
  mi355_stream_t stream_ = nullptr;
  std::string arch_, name_;
  int cus_ = 0;
  size_t totalMem_ = 0;
  std::multimap<size_t, void*> free_;
  std::unordered_map<void*, size_t> sizes_;
  std::unordered_map<std::string, mi355_function_t> kernels_;
  int64_t inUse_ = 0, peak_ = 0, numAllocs_ = 0, largest_ = 0, reserved_ = 0;
  void* pinned_ = nullptr;
};

struct DeviceBuffer {
  void* ptr = nullptr;
  TensorType type;
  bool deleted = false;
  ~DeviceBuffer();
};

struct KindStat {
  int64_t count = 0;
  double ms = 0;
  double flops = 0;
  double bytes = 0;
};

class Executable {
 public:
  explicit Executable(std::unique_ptr<CompiledProgram> prog);
  ~Executable();

  const CompiledProgram& program() const { return *prog_; }
  // Runs the plan on the device stream; returns freshly allocated outputs (enqueued, not awaited).
  // `mayDonate` (optional, one entry per input): the caller allows the program to take that input.  An input the
  // program declares donated (tf.aliasing_output / jax.buffer_donor) and the caller allows is consumed: once the
  // call's work is queued its memory goes back to the allocator (stream order keeps queued readers safe) and the
  // buffer is marked deleted (the reference ignores donation: pjrt_executable.cc:198-246).
  std::vector<std::shared_ptr<DeviceBuffer>> execute(const std::vector<DeviceBuffer*>& inputs, const std::vector<bool>* mayDonate = nullptr);
  // Aggregated step timings (enabled with MI355X_TIMING=<kinds|all>); resolves pending events.
  std::map<std::string, KindStat> timings();
  double compileSeconds = 0;
  int64_t loopHostSyncs() const { return loopSyncs_; }   // host round trips spent reading loop flags so far
  int64_t planGraphLaunches() const { return planGraphLaunches_; }   // execute calls served by one graph launch

 private:
  std::unique_ptr<CompiledProgram> prog_;
  void* arena_ = nullptr;
  void* consts_ = nullptr;
  std::mutex mu_;

  struct Pending { mi355_event_t a, b; std::string kind; double flops, bytes, launches; };
  std::vector<Pending> pending_;
  std::vector<mi355_event_t> eventPool_;
  std::map<std::string, KindStat> stats_;
  std::string timingKinds_;
  int timingEvery_ = 1;
  int timingRepeat_ = 1;
  // Measurement aid (MI355X_TIMING_ROTATE_BYTES=B): the repeated launches of a timed fused kernel cycle through
  // private copies of every buffer of the program (arguments, results, arena), enough of them to hold B bytes, so
  // that no launch finds its operands in a cache left there by the launch before.
  int64_t rotateBytes_ = 0;
  struct ShadowSet { std::vector<void*> params, outs; void* arena = nullptr; };
  std::vector<ShadowSet> shadows_;     // sets 1 .. N-1; set 0 is the call's own buffers
  void prepareShadows(const std::vector<DeviceBuffer*>& in);
  void* resolveIn(const BufRef& r, int set, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) const;
  uint64_t executeCount_ = 0;
  bool timedCall_ = true;

  // Captured bodies of counted loops.  A graph bakes in the addresses of the call's argument and
  // result buffers, so it is kept with a signature of those and rebuilt when they change.
  struct LoopGraph { mi355_graph_t exec = nullptr; uint64_t signature = 0; int64_t itersPerLaunch = 0; uint64_t lastUse = 0; };
  struct LoopGraphs {
    bool scanned = false;
    std::vector<BufRef> external;      // argument / result buffers the body touches
    std::vector<LoopGraph> entries;    // a few recent address sets (buffers recycle through the allocator)
  };
  std::map<const Step*, LoopGraphs> loopGraphs_;
  // The whole plan of a program without loops as one graph (one host call per execute instead of one per launch).
  // Buffers recycle through the allocator, so the address sets of successive calls repeat with a short period: a set is
  // captured the second time it is seen and a few graphs are kept.  Callers whose addresses never repeat keep running
  // launch by launch, and after a number of calls without a single repeat the executable stops looking.
  struct PlanGraph { mi355_graph_t exec = nullptr; uint64_t signature = 0; uint64_t lastUse = 0; };
  std::vector<PlanGraph> planGraphs_;
  std::vector<uint64_t> seenSignatures_;
  bool planGraphsOn_ = false;        // MI355X_PLAN_GRAPHS=1 when the executable was made
  int planGraphState_ = -1;          // -1 not examined, 0 not eligible / given up, 1 eligible
  int64_t planGraphMisses_ = 0, planGraphLaunches_ = 0;
  bool runPlanFromGraph(const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out);
  uint64_t graphClock_ = 0;
  std::map<const Plan*, bool> capturable_;
  bool useGraphs_ = true;
  int64_t hostIteration_ = 0;         // iteration being enqueued of the loop whose counter the host follows (Step::hostCounter)
  bool capturing_ = false;
  bool forkingAllowed_ = true;        // cleared while a plan is captured with everything on one stream
  bool capturable(const Plan& p);
  void runCountedLoop(const Step& s, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out);
  void runDeviceLoop(const Step& s, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out);
  void replayIterations(const Step& s, bool withCond, int64_t count, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out);
  std::map<const Step*, int64_t> lastTrips_;   // iterations each dynamic loop ran on the previous call
  int64_t loopSyncs_ = 0;   // host round trips spent on loop flags (reported by the cost analysis as "loop.host_syncs")

  void loadKernels();
  void* resolve(const BufRef& r, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) const;
  void runPlan(const Plan& plan, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out);
  mi355_stream_t sideStream_ = nullptr;       // second stream for forked steps, created on first use
  mi355_stream_t streamOverride_ = nullptr;   // set while a forked step is being enqueued
  std::vector<mi355_event_t> forkStart_, forkDone_;
  void runStep(const Step& s, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out);
  bool timed(const std::string& kind) const;
  mi355_event_t getEvent();
  void resolvePending();
};

}  // namespace mi355
