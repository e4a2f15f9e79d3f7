// Launch tuning of the grouped GEMM, keyed by problem shape: the counterpart of the reference's tuning
// records (PyTuningRecord / load_tuning_record, src/ths_op/ths_op.cc:208-216), its ProfilingContext
// (include/flux/ths_op/ths_op.h:64-113, src/ths_op/ths_op.cc:217-320) and its TuningConfigRegistry.
// The reference's records pick one of its generated kernel variants; here a record picks the tile
// schedule of the one persistent kernel (height of the raster groups, whether the last round is cut into
// pieces, whether an expert's last row tile may run half height).  No choice changes a result bit.
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

namespace flux_amd {

// What the reference keys on is (UnifiedGemmMeta, RuntimeConfig{m, n, k}); the same facts for this kernel.
struct GemmShapeKey {
  int32_t dtype = 0, nexperts = 0, n = 0, k = 0, max_rows = 0, ngroups = 1;
  auto tie() const { return std::tie(dtype, nexperts, n, k, max_rows, ngroups); }
  bool operator<(const GemmShapeKey &o) const { return tie() < o.tie(); }
  bool operator==(const GemmShapeKey &o) const { return tie() == o.tie(); }
  std::string to_string() const;
};

struct GemmLaunchTuning {
  int32_t raster_rows = 0;  // 0 = the kernel's default
  int32_t sched_flags = 0;  // FLUXMI_SCHED_*
  int32_t reduce_fused = 0;  // layer1 only: 1 = the top-k reduction runs in the GEMM's epilogue, 0 = GEMM, then gather-reduce
  bool operator==(const GemmLaunchTuning &o) const {
    return raster_rows == o.raster_rows && sched_flags == o.sched_flags && reduce_fused == o.reduce_fused;
  }
  std::string to_string() const;
};

struct TuningRecord {
  GemmShapeKey key;
  GemmLaunchTuning best;
  std::string to_string() const;  // one line of the text form read by TuningTable::load_text
};

// Every schedule the profiler tries.
std::vector<GemmLaunchTuning> gemm_tuning_candidates();

// Process-wide table consulted by every grouped-GEMM launch of the ops.
class TuningTable {
 public:
  static TuningTable &instance();
  void add(const GemmShapeKey &key, const GemmLaunchTuning &t);
  std::optional<GemmLaunchTuning> find(const GemmShapeKey &key) const;
  size_t size() const;
  void clear();
  // Text form: one record per line (TuningRecord::to_string); '#' starts a comment.  Returns the number
  // of records read; throws std::runtime_error on a malformed line.
  size_t load_text(const std::string &text);

 private:
  mutable std::mutex mu_;
  std::map<GemmShapeKey, GemmLaunchTuning> table_;
};

class ProfilingContext {
 public:
  static constexpr int kReturnTopK = 5;
  explicit ProfilingContext(std::string name) : name_(std::move(name)) {}
  void add(const GemmShapeKey &key, const GemmLaunchTuning &t, float elapsed_ms);
  GemmLaunchTuning record_best(const GemmShapeKey &key);
  std::string get_code() const;                           // text of all best records (load_text reads it back)
  std::vector<std::string> get_all_prof_results() const;  // per shape: key + the kReturnTopK fastest schedules
  std::string get_latest_prof_result() const;
  TuningRecord get_latest_record() const;
  std::vector<TuningRecord> get_all_records() const;

 private:
  using Ranked = std::map<std::pair<float, int>, GemmLaunchTuning>;  // (ms, insertion order) -> schedule
  std::string topk_string(const Ranked &r) const;
  std::string name_;
  std::map<GemmShapeKey, Ranked> results_;
  std::vector<TuningRecord> best_;
  std::unique_ptr<GemmShapeKey> latest_;
  int counter_ = 0;
};

}  // namespace flux_amd
