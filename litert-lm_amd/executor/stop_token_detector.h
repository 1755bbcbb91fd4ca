// Finds stop-token sequences in the ids a decode loop produces, per batch item
// (runtime/components/stop_token_detector.h, stop_token_detector.cc:40-140):
// a sequence is matched token by token across steps; once an item has stopped,
// every further step is counted so that the caller knows how many trailing
// tokens to drop.
#ifndef LITERT_LM_AMD_EXECUTOR_STOP_TOKEN_DETECTOR_H_
#define LITERT_LM_AMD_EXECUTOR_STOP_TOKEN_DETECTOR_H_

#include <algorithm>
#include <cstddef>
#include <string>
#include <vector>

#include "status.h"

namespace litert::lm {

class StopTokenDetector {
 public:
  explicit StopTokenDetector(size_t batch_size) { ResetBatch(batch_size); }

  // kInvalidArgument for an empty sequence, kAlreadyExists for a repeated one.
  Status AddStopTokenSequence(const std::vector<int>& stop_sequence) {
    if (stop_sequence.empty()) return InvalidArgumentError("Cannot add an empty stop token sequence.");
    if (std::find(sequences_.begin(), sequences_.end(), stop_sequence) != sequences_.end()) {
      std::string text = "{";
      for (size_t i = 0; i < stop_sequence.size(); ++i)
        text += std::to_string(stop_sequence[i]) + (i + 1 < stop_sequence.size() ? ", " : "");
      return AlreadyExistsError("Stop token sequence " + text + "} already exists.");
    }
    sequences_.push_back(stop_sequence);
    for (auto& item : progress_) item.push_back(0);
    return OkStatus();
  }

  // batch_size 0 keeps the current one.
  void ResetBatch(size_t batch_size = 0) {
    const size_t n = batch_size == 0 ? found_.size() : batch_size;
    found_.assign(n, false);
    progress_.assign(n, std::vector<int>(sequences_.size(), 0));
    matched_length_.assign(n, 0);
  }

  // One new token per batch item.
  Status ProcessTokens(const int* latest_tokens, size_t count) {
    if (count != found_.size())
      return InvalidArgumentError("Size of latest_tokens (" + std::to_string(count) +
                                  ") does not match configured batch size (" + std::to_string(found_.size()) + ").");
    if (sequences_.empty())
      return InvalidArgumentError(
          "No stop sequences to check against. Did you forget to call AddStopTokenSequence()?");
    for (size_t i = 0; i < count; ++i) {
      if (found_[i]) {
        ++matched_length_[i];  // already stopped: one more trailing step
        continue;
      }
      const int token = latest_tokens[i];
      for (size_t k = 0; k < sequences_.size(); ++k) {
        const std::vector<int>& seq = sequences_[k];
        int& matched = progress_[i][k];
        if (matched < static_cast<int>(seq.size()) && seq[matched] == token) ++matched;
        else matched = seq[0] == token ? 1 : 0;  // restart, possibly on this very token
        if (matched > 0 && matched == static_cast<int>(seq.size())) {
          found_[i] = true;
          matched_length_[i] = static_cast<int>(seq.size());
        }
      }
    }
    return OkStatus();
  }
  Status ProcessTokens(const std::vector<int>& latest_tokens) {
    return ProcessTokens(latest_tokens.data(), latest_tokens.size());
  }

  // Per item: length of the matched sequence plus the steps taken since.
  const std::vector<int>& GetStepsBeforeStopTokens() const { return matched_length_; }
  const std::vector<bool>& GetStopTokensFound() const { return found_; }

  StatusOr<bool> AllDone() const {
    if (found_.empty()) return FailedPreconditionError("The Detector is not initialized with non-zero batch size.");
    return std::all_of(found_.begin(), found_.end(), [](bool f) { return f; });
  }

 private:
  std::vector<std::vector<int>> sequences_;
  std::vector<std::vector<int>> progress_;  // [item][sequence] tokens matched so far
  std::vector<bool> found_;
  std::vector<int> matched_length_;
};

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_STOP_TOKEN_DETECTOR_H_
