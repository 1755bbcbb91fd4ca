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

namespace {
struct SectionWords {
  const char* noun;         // in the error texts
  const char* label_stem;   // of a turn label, null for named rows
};
const SectionWords& Words(BenchmarkInfo::Section s) {
  static const SectionWords kWords[] = {{"Phase", nullptr}, {"Prefill turn", "prefill:"}, {"Decode turn", "decode:"},
                                        {"Mark", nullptr}};
  return kWords[static_cast<int>(s)];
}
}  // namespace

std::string BenchmarkInfo::TurnLabel(Section section) const {
  return Words(section).label_stem + std::to_string(Count(section));
}

BenchmarkInfo::Row* BenchmarkInfo::Find(Section section, const std::string& label) {
  const bool mark = section == Section::kMark;
  for (Row& row : rows_)
    if ((row.section == Section::kMark) == mark && row.label == label) return &row;
  return nullptr;
}

Status BenchmarkInfo::Start(Section section, const std::string& label) {
  if (Find(section, label) != nullptr)
    return InternalError(std::string(Words(section).noun) + " " + label + " already started.");
  rows_.push_back(Row{section, label, Now()});
  return OkStatus();
}

Status BenchmarkInfo::Stop(Section section, const std::string& label, uint64_t tokens) {
  const TimePoint now = Now();
  Row* row = Find(section, label);
  if (row == nullptr) return InternalError(std::string(Words(section).noun) + " " + label + " not started.");
  // A phase may be ended again: the later reading replaces the earlier one. The row counts for the section that
  // ends it (which only differs from the one that started it when a phase was named like a turn).
  row->section = section;
  row->took = std::chrono::duration_cast<Duration>(now - row->since);
  row->tokens = tokens;
  row->measured = true;
  return OkStatus();
}

Status BenchmarkInfo::TimeMarkDelta(const std::string& mark_name) {
  const TimePoint now = Now();
  if (Row* row = Find(Section::kMark, mark_name)) {
    row->took = std::chrono::duration_cast<Duration>(now - row->since);
    row->measured = true;
    row->since = now;
  } else {
    rows_.push_back(Row{Section::kMark, mark_name, now});
  }
  return OkStatus();
}

std::map<std::string, Duration> BenchmarkInfo::Named(Section section) const {
  std::map<std::string, Duration> out;
  for (const Row& row : rows_)
    if (row.section == section && row.measured) out[row.label] = row.took;
  return out;
}

uint64_t BenchmarkInfo::Count(Section section) const {
  uint64_t n = 0;
  for (const Row& row : rows_) n += row.section == section && row.measured;
  return n;
}

const BenchmarkInfo::Row* BenchmarkInfo::TurnRow(Section section, int turn_index) const {
  if (turn_index < 0) return nullptr;
  for (const Row& row : rows_)
    if (row.section == section && row.measured && turn_index-- == 0) return &row;
  return nullptr;
}

BenchmarkTurnData BenchmarkInfo::Turn(Section section, int turn_index) const {
  const Row* row = TurnRow(section, turn_index);
  return row ? BenchmarkTurnData(row->tokens, row->took) : BenchmarkTurnData(0, Duration::zero());
}

double BenchmarkInfo::TokensPerSec(Section section, int turn_index) const {
  const Row* row = TurnRow(section, turn_index);
  if (row == nullptr || row->took <= Duration::zero()) return 0.0;
  const double seconds = static_cast<double>(row->took.count()) * 1e-9;
  return seconds > 0.0 ? static_cast<double>(row->tokens) / seconds : 0.0;
}

std::ostream& operator<<(std::ostream& os, const BenchmarkTurnData& data) {
  return os << "Processed " << data.num_tokens << " tokens in " << FormatDuration(data.duration) << " duration.\n"
            << std::flush;
}

// The report, section by section, in the reference's wording (io_types.cc:255-308): two decimals throughout,
// a rule after every section, the marks only when there are any.
std::ostream& operator<<(std::ostream& os, const BenchmarkInfo& info) {
  static const char kRule[] = "--------------------------------------------------\n";
  os << std::fixed << std::setprecision(2) << "BenchmarkInfo:\n";

  const auto phases = info.GetInitPhases();
  os << "  Init Phases (" << phases.size() << "):\n";
  double total_ms = 0.0;
  for (const auto& [name, took] : phases) {
    total_ms += Millis(took);
    os << "    - " << name << ": " << Millis(took) << " ms\n";
  }
  if (phases.empty()) os << "    No init phases recorded.\n";
  else os << "    Total init time: " << total_ms << " ms\n";
  os << kRule;

  struct TurnSection {
    const char* title;
    const char* lower;
    uint64_t turns;
    BenchmarkTurnData (BenchmarkInfo::*turn)(int) const;
    double (BenchmarkInfo::*speed)(int) const;
  };
  const TurnSection sections[] = {
      {"Prefill", "prefill", info.GetTotalPrefillTurns(), &BenchmarkInfo::GetPrefillTurn,
       &BenchmarkInfo::GetPrefillTokensPerSec},
      {"Decode", "decode", info.GetTotalDecodeTurns(), &BenchmarkInfo::GetDecodeTurn,
       &BenchmarkInfo::GetDecodeTokensPerSec}};
  for (const TurnSection& s : sections) {
    os << "  " << s.title << " Turns (Total: " << s.turns << "):\n";
    if (s.turns == 0) os << "    No " << s.lower << " turns recorded.\n";
    for (uint64_t i = 0; i < s.turns; ++i) {
      const int turn = static_cast<int>(i);
      os << "    " << s.title << " Turn " << i + 1 << ": " << (info.*s.turn)(turn);
      os << "      " << s.title << " Speed: " << (info.*s.speed)(turn) << " tokens/sec.\n";
    }
    os << kRule;
  }

  const auto marks = info.GetMarkDurations();
  if (!marks.empty()) os << "  Mark Durations (" << marks.size() << "):\n";
  for (const auto& [name, took] : marks) os << "    - " << name << ": " << FormatDuration(took) << "\n";
  return os << kRule << std::flush;
}

}  // namespace litert::lm
