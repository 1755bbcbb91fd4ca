// Timing record of a benchmark run, reported in the reference's format
// (runtime/engine/io_types.h:86-163, io_types.cc:100-308) so that numbers of
// this build can be laid beside the reference's `litert_lm_main --benchmark`
// output (README.md:390-400: 1024 prefill tokens, 256 decode tokens).
//
// Everything timed is a row of one table: a section (init phase, prefill turn,
// decode turn, mark), a label, when its clock last started and what it
// measured. The reference's entry points are the thin methods below; what they
// promise is kept: a phase or turn starts once and ends only after it started
// (kInternal otherwise, with the reference's texts), turns are labelled
// "prefill:N" / "decode:N" in the same label space as the init phases, and a
// mark measures the time between its two latest calls.
//
// Durations are std::chrono::nanoseconds; FormatDuration restates how
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
  enum class Section { kInitPhase, kPrefillTurn, kDecodeTurn, kMark };

  explicit BenchmarkInfo(const BenchmarkParams& params) : params_(params) {}
  const BenchmarkParams& GetBenchmarkParams() const { return params_; }

  Status TimeInitPhaseStart(const std::string& phase_name) { return Start(Section::kInitPhase, phase_name); }
  Status TimeInitPhaseEnd(const std::string& phase_name) { return Stop(Section::kInitPhase, phase_name, 0); }
  Status TimePrefillTurnStart() { return Start(Section::kPrefillTurn, TurnLabel(Section::kPrefillTurn)); }
  Status TimePrefillTurnEnd(uint64_t num_prefill_tokens) {
    return Stop(Section::kPrefillTurn, TurnLabel(Section::kPrefillTurn), num_prefill_tokens);
  }
  Status TimeDecodeTurnStart() { return Start(Section::kDecodeTurn, TurnLabel(Section::kDecodeTurn)); }
  Status TimeDecodeTurnEnd(uint64_t num_decode_tokens) {
    return Stop(Section::kDecodeTurn, TurnLabel(Section::kDecodeTurn), num_decode_tokens);
  }
  // The time between the two latest calls with the same name.
  Status TimeMarkDelta(const std::string& mark_name);

  // Measured rows of a section: name -> duration (init phases, marks), or in turn order (turns).
  std::map<std::string, Duration> GetInitPhases() const { return Named(Section::kInitPhase); }
  std::map<std::string, Duration> GetMarkDurations() const { return Named(Section::kMark); }
  uint64_t GetTotalPrefillTurns() const { return Count(Section::kPrefillTurn); }
  uint64_t GetTotalDecodeTurns() const { return Count(Section::kDecodeTurn); }
  BenchmarkTurnData GetPrefillTurn(int turn_index) const { return Turn(Section::kPrefillTurn, turn_index); }
  BenchmarkTurnData GetDecodeTurn(int turn_index) const { return Turn(Section::kDecodeTurn, turn_index); }
  // 0 for a turn that does not exist or took no time.
  double GetPrefillTokensPerSec(int turn_index) const { return TokensPerSec(Section::kPrefillTurn, turn_index); }
  double GetDecodeTokensPerSec(int turn_index) const { return TokensPerSec(Section::kDecodeTurn, turn_index); }

 private:
  struct Row {
    Section section;
    std::string label;
    TimePoint since;        // when the clock of this row last started
    bool measured = false;  // `took` (and `tokens`) hold a result
    Duration took{0};
    uint64_t tokens = 0;
  };
  static TimePoint Now() { return std::chrono::steady_clock::now(); }
  // "prefill:N" / "decode:N", N = turns of that section measured so far.
  std::string TurnLabel(Section section) const;
  // Phases and turns share their labels (a phase called "prefill:0" is the first prefill turn's clock); marks do not.
  Row* Find(Section section, const std::string& label);
  const Row* TurnRow(Section section, int turn_index) const;
  Status Start(Section section, const std::string& label);
  Status Stop(Section section, const std::string& label, uint64_t tokens);
  std::map<std::string, Duration> Named(Section section) const;
  uint64_t Count(Section section) const;
  BenchmarkTurnData Turn(Section section, int turn_index) const;
  double TokensPerSec(Section section, int turn_index) const;

  BenchmarkParams params_;
  std::vector<Row> rows_;  // in order of first start
};
std::ostream& operator<<(std::ostream& os, const BenchmarkInfo& info);

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_BENCHMARK_INFO_H_
