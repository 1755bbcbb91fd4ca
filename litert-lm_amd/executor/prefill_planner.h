// Prefill chunk planning over the static sequence lengths of the prefill
// runners: the longest runner while a full one fits, then one call on the
// shortest runner that still holds the remainder. Same plan as
// GetOptimizedPrefillWorkGroups in
// runtime/executor/litert_compiled_model_executor_utils.cc:300-330.
#ifndef LITERT_LM_AMD_EXECUTOR_PREFILL_PLANNER_H_
#define LITERT_LM_AMD_EXECUTOR_PREFILL_PLANNER_H_

#include <functional>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "status.h"

namespace litert::lm {

// Runner length -> signature name, longest first
// (runtime/executor/litert_compiled_model_executor_utils.h:37-38).
using SortedPrefillSignatureMap = std::map<int, std::string, std::greater<int>>;

inline StatusOr<std::vector<std::pair<std::string, int>>> GetOptimizedPrefillWorkGroups(
    const SortedPrefillSignatureMap& runners, int input_length) {
  if (runners.empty()) return FailedPreconditionError("No prefill runner available.");
  std::vector<std::pair<std::string, int>> groups;
  const auto& longest = *runners.begin();
  for (; input_length >= longest.first; input_length -= longest.first) groups.emplace_back(longest.second, longest.first);
  if (input_length > 0) {
    // walk from the longest runner down and stop at the last one that still fits
    auto pick = runners.begin();
    for (auto it = runners.begin(); it != runners.end() && it->first >= input_length; ++it) pick = it;
    groups.emplace_back(pick->second, input_length);
  }
  return groups;
}

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_PREFILL_PLANNER_H_
