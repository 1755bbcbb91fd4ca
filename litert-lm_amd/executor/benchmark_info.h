// Timing record of a benchmark run in the reference's own report format
// (runtime/engine/io_types.h:86-163, io_types.cc:100-308): init phases,
// prefill / decode turns with tokens per second, mark-to-mark durations, and
// the text the reference's `operator<<` prints, so that numbers of this build
// can be laid beside the reference's `litert_lm_main --benchmark` output
// (README.md:390-400: 1024 prefill tokens, 256 decode tokens).
//
// Durations are std::chrono::nanoseconds here; FormatDuration restates how
// absl::Duration (a dependency the reference does not vendor) prints itself
// ("1.5ms", "2m3.25s"): the reference's test matches that part of the text with
// `.*` only (io_types_test.cc:255-272), so the digits are not pinned by it.
#ifndef LITERT_LM_AMD_EXECUTOR_BENCHMARK_INFO_H_
#define LITERT_LM_AMD_EXECUTOR_BENCHMARK_INFO_H_

#include <chrono>
#include <cstdint>
#include <map>
#include <ostream>
#include <string>
#include <vector>

#include "status.h"

namespace litert::lm {

using Duration = std::chrono::nanoseconds;
using TimePoint = std::chrono::steady_clock::time_point;

// proto::BenchmarkParams (runtime/proto/engine.proto): 0 = not forced.
struct BenchmarkParams {
  int num_prefill_tokens = 0;
  int num_decode_tokens = 0;
};

std::string FormatDuration(Duration d);

struct BenchmarkTurnData {
  BenchmarkTurnData(uint64_t tokens, Duration dur) : duration(dur), num_tokens(tokens) {}
  Duration duration;
  uint64_t num_tokens;
};
std::ostream& operator<<(std::ostream& os, const BenchmarkTurnData& data);

class BenchmarkInfo {
 public:
  explicit BenchmarkInfo(const BenchmarkParams& params) : params_(params) {}
  const BenchmarkParams& GetBenchmarkParams() const { return params_; }

  // A phase / turn may be started once and ended only after its start: kInternal otherwise.
  Status TimeInitPhaseStart(const std::string& phase_name);
  Status TimeInitPhaseEnd(const std::string& phase_name);
  Status TimePrefillTurnStart();
  Status TimePrefillTurnEnd(uint64_t num_prefill_tokens);
  Status TimeDecodeTurnStart();
  Status TimeDecodeTurnEnd(uint64_t num_decode_tokens);
  // The time between the two latest calls with the same name.
  Status TimeMarkDelta(const std::string& mark_name);

  const std::map<std::string, Duration>& GetInitPhases() const { return init_phases_; }
  const std::map<std::string, Duration>& GetMarkDurations() const { return mark_durations_; }
  uint64_t GetTotalPrefillTurns() const { return prefill_turns_.size(); }
  const BenchmarkTurnData& GetPrefillTurn(int turn_index) const { return prefill_turns_[turn_index]; }
  double GetPrefillTokensPerSec(int turn_index) const;
  uint64_t GetTotalDecodeTurns() const { return decode_turns_.size(); }
  const BenchmarkTurnData& GetDecodeTurn(int turn_index) const { return decode_turns_[turn_index]; }
  double GetDecodeTokensPerSec(int turn_index) const;

 private:
  static TimePoint Now() { return std::chrono::steady_clock::now(); }
  static double TokensPerSec(const std::vector<BenchmarkTurnData>& turns, int turn_index);
  BenchmarkParams params_;
  std::map<std::string, TimePoint> start_time_map_;
  std::map<std::string, TimePoint> mark_time_map_;
  int prefill_turn_index_ = 0;
  int decode_turn_index_ = 0;
  std::map<std::string, Duration> init_phases_;
  std::map<std::string, Duration> mark_durations_;
  std::vector<BenchmarkTurnData> prefill_turns_;
  std::vector<BenchmarkTurnData> decode_turns_;
};
std::ostream& operator<<(std::ostream& os, const BenchmarkInfo& info);

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_BENCHMARK_INFO_H_
