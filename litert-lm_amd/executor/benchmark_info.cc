#include "benchmark_info.h"

#include <cmath>
#include <cstdio>
#include <iomanip>

namespace litert::lm {
namespace {

// One "<number><unit>" piece of a duration with up to `digits` decimals,
// trailing zeros dropped; nothing at all for a zero value.
void AppendNumberUnit(std::string* out, double value, const char* unit, int digits) {
  double int_part = 0.0;
  const double scale = std::pow(10.0, digits);
  int64_t frac = static_cast<int64_t>(std::llround(std::modf(value, &int_part) * scale));
  if (frac >= static_cast<int64_t>(scale)) {  // .9999.. rounded up
    frac -= static_cast<int64_t>(scale);
    int_part += 1.0;
  }
  if (int_part == 0.0 && frac == 0) return;
  char buf[64];
  snprintf(buf, sizeof(buf), "%lld", static_cast<long long>(int_part));
  out->append(buf);
  if (frac != 0) {
    snprintf(buf, sizeof(buf), "%0*lld", digits, static_cast<long long>(frac));
    std::string f(buf);
    while (!f.empty() && f.back() == '0') f.pop_back();
    out->push_back('.');
    out->append(f);
  }
  out->append(unit);
}

double Millis(Duration d) { return static_cast<double>(d.count()) * 1e-6; }

}  // namespace

// Below one second the largest of ns / us / ms that keeps the value >= 1, with
// decimals down to the nanosecond; from one second on hours, minutes and
// seconds ("1h2m3.5s"), zero-valued units left out; "0" for nothing.
std::string FormatDuration(Duration d) {
  std::string s;
  int64_t ns = d.count();
  if (ns < 0) {
    s = "-";
    ns = -ns;
  }
  if (ns < 1000000000LL) {
    if (ns < 1000) AppendNumberUnit(&s, static_cast<double>(ns), "ns", 2);
    else if (ns < 1000000) AppendNumberUnit(&s, ns / 1e3, "us", 5);
    else AppendNumberUnit(&s, ns / 1e6, "ms", 8);
  } else {
    const int64_t hours = ns / 3600000000000LL;
    ns -= hours * 3600000000000LL;
    const int64_t minutes = ns / 60000000000LL;
    ns -= minutes * 60000000000LL;
    if (hours) s += std::to_string(hours) + "h";
    if (minutes) s += std::to_string(minutes) + "m";
    AppendNumberUnit(&s, ns / 1e9, "s", 11);
  }
  if (s.empty() || s == "-") s = "0";
  return s;
}

Status BenchmarkInfo::TimeInitPhaseStart(const std::string& phase_name) {
  if (start_time_map_.count(phase_name)) return InternalError("Phase " + phase_name + " already started.");
  start_time_map_[phase_name] = Now();
  return OkStatus();
}

Status BenchmarkInfo::TimeInitPhaseEnd(const std::string& phase_name) {
  if (!start_time_map_.count(phase_name)) return InternalError("Phase " + phase_name + " not started.");
  init_phases_[phase_name] = std::chrono::duration_cast<Duration>(Now() - start_time_map_[phase_name]);
  return OkStatus();
}

Status BenchmarkInfo::TimeMarkDelta(const std::string& mark_name) {
  const TimePoint now = Now();
  auto it = mark_time_map_.find(mark_name);
  if (it != mark_time_map_.end()) mark_durations_[mark_name] = std::chrono::duration_cast<Duration>(now - it->second);
  mark_time_map_[mark_name] = now;
  return OkStatus();
}

Status BenchmarkInfo::TimePrefillTurnStart() {
  const std::string phase_name = "prefill:" + std::to_string(prefill_turn_index_);
  if (start_time_map_.count(phase_name)) return InternalError("Prefill turn " + phase_name + " already started.");
  start_time_map_[phase_name] = Now();
  return OkStatus();
}

Status BenchmarkInfo::TimePrefillTurnEnd(uint64_t num_prefill_tokens) {
  const std::string phase_name = "prefill:" + std::to_string(prefill_turn_index_);
  if (!start_time_map_.count(phase_name)) return InternalError("Prefill turn " + phase_name + " not started.");
  prefill_turns_.emplace_back(num_prefill_tokens, std::chrono::duration_cast<Duration>(Now() - start_time_map_[phase_name]));
  prefill_turn_index_++;
  return OkStatus();
}

Status BenchmarkInfo::TimeDecodeTurnStart() {
  const std::string phase_name = "decode:" + std::to_string(decode_turn_index_);
  if (start_time_map_.count(phase_name)) return InternalError("Decode turn " + phase_name + " already started.");
  start_time_map_[phase_name] = Now();
  return OkStatus();
}

Status BenchmarkInfo::TimeDecodeTurnEnd(uint64_t num_decode_tokens) {
  const std::string phase_name = "decode:" + std::to_string(decode_turn_index_);
  if (!start_time_map_.count(phase_name)) return InternalError("Decode turn " + phase_name + " not started.");
  decode_turns_.emplace_back(num_decode_tokens, std::chrono::duration_cast<Duration>(Now() - start_time_map_[phase_name]));
  decode_turn_index_++;
  return OkStatus();
}

double BenchmarkInfo::TokensPerSec(const std::vector<BenchmarkTurnData>& turns, int turn_index) {
  if (turn_index < 0 || static_cast<size_t>(turn_index) >= turns.size()) return 0.0;
  const BenchmarkTurnData& turn = turns[turn_index];
  if (turn.duration <= Duration::zero()) return 0.0;
  const double seconds = static_cast<double>(turn.duration.count()) * 1e-9;
  if (seconds <= 0.0) return 0.0;
  return static_cast<double>(turn.num_tokens) / seconds;
}

double BenchmarkInfo::GetPrefillTokensPerSec(int turn_index) const { return TokensPerSec(prefill_turns_, turn_index); }
double BenchmarkInfo::GetDecodeTokensPerSec(int turn_index) const { return TokensPerSec(decode_turns_, turn_index); }

std::ostream& operator<<(std::ostream& os, const BenchmarkTurnData& data) {
  os << "Processed " << data.num_tokens << " tokens in " << FormatDuration(data.duration) << " duration." << std::endl;
  return os;
}

std::ostream& operator<<(std::ostream& os, const BenchmarkInfo& info) {
  os << std::fixed << std::setprecision(2);
  os << "BenchmarkInfo:" << std::endl;
  os << "  Init Phases (" << info.GetInitPhases().size() << "):" << std::endl;
  if (info.GetInitPhases().empty()) {
    os << "    No init phases recorded." << std::endl;
  } else {
    double total_time = 0.0;
    for (const auto& phase : info.GetInitPhases()) {
      total_time += Millis(phase.second);
      os << "    - " << phase.first << ": " << Millis(phase.second) << " ms" << std::endl;
    }
    os << "    Total init time: " << total_time << " ms" << std::endl;
  }
  os << "--------------------------------------------------" << std::endl;
  os << "  Prefill Turns (Total: " << info.GetTotalPrefillTurns() << "):" << std::endl;
  if (info.GetTotalPrefillTurns() == 0) {
    os << "    No prefill turns recorded." << std::endl;
  } else {
    for (uint64_t i = 0; i < info.GetTotalPrefillTurns(); ++i) {
      os << "    Prefill Turn " << i + 1 << ": " << info.GetPrefillTurn(static_cast<int>(i));
      os << "      Prefill Speed: " << info.GetPrefillTokensPerSec(static_cast<int>(i)) << " tokens/sec." << std::endl;
    }
  }
  os << "--------------------------------------------------" << std::endl;
  os << "  Decode Turns (Total: " << info.GetTotalDecodeTurns() << "):" << std::endl;
  if (info.GetTotalDecodeTurns() == 0) {
    os << "    No decode turns recorded." << std::endl;
  } else {
    for (uint64_t i = 0; i < info.GetTotalDecodeTurns(); ++i) {
      os << "    Decode Turn " << i + 1 << ": " << info.GetDecodeTurn(static_cast<int>(i));
      os << "      Decode Speed: " << info.GetDecodeTokensPerSec(static_cast<int>(i)) << " tokens/sec." << std::endl;
    }
  }
  os << "--------------------------------------------------" << std::endl;
  if (!info.GetMarkDurations().empty()) {
    os << "  Mark Durations (" << info.GetMarkDurations().size() << "):" << std::endl;
    for (const auto& mark : info.GetMarkDurations())
      os << "    - " << mark.first << ": " << FormatDuration(mark.second) << std::endl;
  }
  os << "--------------------------------------------------" << std::endl;
  return os;
}

}  // namespace litert::lm
