// Shape-keyed launch tuning of the grouped GEMM: table, text form and profiling records.
#include "tuning.h"

#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iomanip>
#include <sstream>
#include <stdexcept>

#include "fluxmi.h"

namespace flux_amd {

std::string GemmShapeKey::to_string() const {
  std::ostringstream ss;
  ss << "dtype=" << (dtype == FLUXMI_BF16 ? "bf16" : (dtype == FLUXMI_FP16 ? "f16" : "e4m3")) << " experts=" << nexperts << " n=" << n << " k=" << k
     << " rows=" << max_rows << " groups=" << ngroups;
  return ss.str();
}

std::string GemmLaunchTuning::to_string() const {
  std::ostringstream ss;
  ss << "raster_rows=" << raster_rows << " sched_flags=" << sched_flags;
  if (reduce_fused) ss << " reduce=fused";
  return ss.str();
}

std::string TuningRecord::to_string() const { return "fluxmi_gemm_tuning " + key.to_string() + " " + best.to_string(); }

std::vector<GemmLaunchTuning> gemm_tuning_candidates() {
  std::vector<GemmLaunchTuning> out;
  for (int32_t flags : {0, FLUXMI_SCHED_WHOLE_TAIL_TILES, FLUXMI_SCHED_NO_HALF_TILES,
                        FLUXMI_SCHED_WHOLE_TAIL_TILES | FLUXMI_SCHED_NO_HALF_TILES})
    for (int32_t rows : {8, 4, 16}) out.push_back(GemmLaunchTuning{rows, flags});
  // where the few last rows of an expert run: as 64 x 64 pieces behind all other tiles, or in place
  out.push_back(GemmLaunchTuning{8, FLUXMI_SCHED_NO_SKINNY_TAIL});
  out.push_back(GemmLaunchTuning{8, FLUXMI_SCHED_FORCE_SKINNY_TAIL});
  // both forms of the ring fills, whatever the default picks for the shape
  out.push_back(GemmLaunchTuning{8, FLUXMI_SCHED_HALF_LINE_FILLS});
  out.push_back(GemmLaunchTuning{8, FLUXMI_SCHED_WHOLE_LINE_FILLS});
  return out;
}

TuningTable &TuningTable::instance() {
  static TuningTable *table = [] {
    auto *t = new TuningTable();
    // Records written by ProfilingContext::get_code(), loaded once per process.
    if (const char *path = std::getenv("FLUX_AMD_TUNING_FILE")) {
      std::ifstream f(path);
      if (!f) throw std::runtime_error(std::string("FLUX_AMD_TUNING_FILE: cannot open ") + path);
      std::stringstream ss;
      ss << f.rdbuf();
      t->load_text(ss.str());
    }
    return t;
  }();
  return *table;
}

void TuningTable::add(const GemmShapeKey &key, const GemmLaunchTuning &t) {
  std::lock_guard<std::mutex> lock(mu_);
  table_[key] = t;
}

std::optional<GemmLaunchTuning> TuningTable::find(const GemmShapeKey &key) const {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = table_.find(key);
  if (it == table_.end()) return std::nullopt;
  return it->second;
}

size_t TuningTable::size() const {
  std::lock_guard<std::mutex> lock(mu_);
  return table_.size();
}

void TuningTable::clear() {
  std::lock_guard<std::mutex> lock(mu_);
  table_.clear();
}

size_t TuningTable::load_text(const std::string &text) {
  std::istringstream in(text);
  std::string line;
  size_t count = 0;
  int lineno = 0;
  while (std::getline(in, line)) {
    ++lineno;
    const size_t hash = line.find('#');
    if (hash != std::string::npos) line.resize(hash);
    std::istringstream ls(line);
    std::string word;
    if (!(ls >> word)) continue;  // blank
    auto fail = [&](const std::string &why) {
      throw std::runtime_error("tuning text line " + std::to_string(lineno) + ": " + why);
    };
    if (word != "fluxmi_gemm_tuning") fail("expected 'fluxmi_gemm_tuning', got '" + word + "'");
    GemmShapeKey key;
    GemmLaunchTuning t;
    int seen = 0;
    while (ls >> word) {
      const size_t eq = word.find('=');
      if (eq == std::string::npos) fail("expected name=value, got '" + word + "'");
      const std::string name = word.substr(0, eq), value = word.substr(eq + 1);
      if (name == "dtype") {
        if (value == "bf16") key.dtype = FLUXMI_BF16;
        else if (value == "e4m3") key.dtype = FLUXMI_FP8_E4M3;
        else if (value == "f16") key.dtype = FLUXMI_FP16;
        else fail("unknown dtype '" + value + "'");
        seen |= 1;
        continue;
      }
      if (name == "reduce") {  // optional: the form of layer1's top-k reduction
        if (value == "fused") t.reduce_fused = 1;
        else if (value == "twopass") t.reduce_fused = 0;
        else fail("unknown reduce form '" + value + "'");
        continue;
      }
      char *end = nullptr;
      const long v = std::strtol(value.c_str(), &end, 10);
      if (value.empty() || *end != '\0' || v < 0 || v > 0x7fffffffl) fail("bad number in '" + word + "'");
      if (name == "experts") key.nexperts = static_cast<int32_t>(v), seen |= 2;
      else if (name == "n") key.n = static_cast<int32_t>(v), seen |= 4;
      else if (name == "k") key.k = static_cast<int32_t>(v), seen |= 8;
      else if (name == "rows") key.max_rows = static_cast<int32_t>(v), seen |= 16;
      else if (name == "groups") key.ngroups = static_cast<int32_t>(v), seen |= 32;
      else if (name == "raster_rows") t.raster_rows = static_cast<int32_t>(v), seen |= 64;
      else if (name == "sched_flags") t.sched_flags = static_cast<int32_t>(v), seen |= 128;
      else fail("unknown field '" + name + "'");
    }
    if (seen != 255) fail("missing fields");
    if (t.raster_rows > 1024 || (t.sched_flags & ~(FLUXMI_SCHED_WHOLE_TAIL_TILES | FLUXMI_SCHED_NO_HALF_TILES | FLUXMI_SCHED_NO_SKINNY_TAIL |
                                                  FLUXMI_SCHED_FORCE_SKINNY_TAIL | FLUXMI_SCHED_HALF_LINE_FILLS | FLUXMI_SCHED_WHOLE_LINE_FILLS)))
      fail("raster_rows / sched_flags out of range");
    add(key, t);
    ++count;
  }
  return count;
}

void ProfilingContext::add(const GemmShapeKey &key, const GemmLaunchTuning &t, float elapsed_ms) {
  results_[key].emplace(std::make_pair(elapsed_ms, counter_++), t);
}

GemmLaunchTuning ProfilingContext::record_best(const GemmShapeKey &key) {
  auto it = results_.find(key);
  if (it == results_.end() || it->second.empty())
    throw std::runtime_error("ProfilingContext: no prof results found for " + key.to_string());
  latest_ = std::make_unique<GemmShapeKey>(key);
  const GemmLaunchTuning best = it->second.begin()->second;
  bool replaced = false;
  for (auto &r : best_)
    if (r.key == key) r.best = best, replaced = true;
  if (!replaced) best_.push_back(TuningRecord{key, best});
  return best;
}

std::string ProfilingContext::topk_string(const Ranked &r) const {
  std::ostringstream ss;
  int idx = 0;
  for (auto it = r.begin(); idx < kReturnTopK && it != r.end(); ++it) {
    ss << " * TopK=" << (++idx) << std::setprecision(3) << " (" << it->first.first << " ms): " << it->second.to_string();
    if (idx < kReturnTopK) ss << "\n";
  }
  return ss.str();
}

std::string ProfilingContext::get_code() const {
  std::ostringstream ss;
  ss << "# grouped GEMM launch tuning, profiling context '" << name_ << "'\n";
  for (const auto &r : best_) ss << r.to_string() << "\n";
  return ss.str();
}

std::vector<std::string> ProfilingContext::get_all_prof_results() const {
  std::vector<std::string> out;
  for (const auto &kv : results_) out.push_back(kv.first.to_string() + "\n" + topk_string(kv.second));
  return out;
}

std::string ProfilingContext::get_latest_prof_result() const {
  if (!latest_) throw std::runtime_error("ProfilingContext: no latest prof results found");
  return latest_->to_string() + "\n" + topk_string(results_.at(*latest_));
}

TuningRecord ProfilingContext::get_latest_record() const {
  if (!latest_) throw std::runtime_error("ProfilingContext: no latest prof results found");
  return TuningRecord{*latest_, results_.at(*latest_).begin()->second};
}

std::vector<TuningRecord> ProfilingContext::get_all_records() const {
  std::vector<TuningRecord> out;
  for (const auto &kv : results_) out.push_back(TuningRecord{kv.first, kv.second.begin()->second});
  return out;
}

}  // namespace flux_amd
