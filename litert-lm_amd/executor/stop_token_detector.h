// Finds stop-token sequences in the ids a decode loop produces, one id per
// batch item and step. Behaviour of runtime/components/stop_token_detector.h
// (stop_token_detector.cc:40-140), built here from two small parts:
//
//  * StopSequence is the matcher of one stop sequence: a cursor says how many
//    of its tokens the latest ids of an item have matched, Advance() moves it by
//    one id. On a mismatch the cursor does not fall back to the longest border
//    (no KMP): it restarts at 1 when the id is the sequence's first token, else
//    at 0, which is what the reference does. Against the sequence "1 1 2" the
//    ids "1 1 1 2" therefore do not complete (the third 1 restarts the cursor
//    at 1, not at 2), while "1 2 1 2 3" against "1 2 3" does.
//  * Lane is the state of one batch item: a cursor per sequence, and once a
//    sequence has completed, the count the caller uses to drop trailing ids:
//    the completed sequence's length plus one per further step.
#ifndef LITERT_LM_AMD_EXECUTOR_STOP_TOKEN_DETECTOR_H_
#define LITERT_LM_AMD_EXECUTOR_STOP_TOKEN_DETECTOR_H_

#include <cstddef>
#include <string>
#include <utility>
#include <vector>

#include "status.h"

namespace litert::lm {

class StopSequence {
 public:
  explicit StopSequence(std::vector<int> ids) : ids_(std::move(ids)) {}
  const std::vector<int>& ids() const { return ids_; }
  int length() const { return static_cast<int>(ids_.size()); }
  // The cursor after `id`; length() means the sequence has just completed.
  int Advance(int cursor, int id) const {
    if (cursor < length() && ids_[cursor] == id) return cursor + 1;
    return ids_.front() == id ? 1 : 0;
  }
  std::string Text() const {
    std::string text = "{";
    for (size_t i = 0; i < ids_.size(); ++i) text += (i ? ", " : "") + std::to_string(ids_[i]);
    return text + "}";
  }

 private:
  std::vector<int> ids_;  // never empty
};

class StopTokenDetector {
 public:
  explicit StopTokenDetector(size_t batch_size) { ResetBatch(batch_size); }

  // kInvalidArgument for an empty sequence, kAlreadyExists for a repeated one.
  Status AddStopTokenSequence(const std::vector<int>& stop_sequence) {
    if (stop_sequence.empty()) return InvalidArgumentError("Cannot add an empty stop token sequence.");
    for (const StopSequence& known : sequences_)
      if (known.ids() == stop_sequence)
        return AlreadyExistsError("Stop token sequence " + known.Text() + " already exists.");
    sequences_.emplace_back(stop_sequence);
    for (Lane& lane : lanes_) lane.cursors.push_back(0);
    Publish();
    return OkStatus();
  }

  // Forgets all progress; batch_size 0 keeps the current one.
  void ResetBatch(size_t batch_size = 0) {
    lanes_.assign(batch_size == 0 ? lanes_.size() : batch_size, Lane{std::vector<int>(sequences_.size(), 0), 0, false});
    Publish();
  }

  // One new id per batch item.
  Status ProcessTokens(const int* latest_tokens, size_t count) {
    if (count != lanes_.size())
      return InvalidArgumentError("Size of latest_tokens (" + std::to_string(count) +
                                  ") does not match configured batch size (" + std::to_string(lanes_.size()) + ").");
    if (sequences_.empty())
      return InvalidArgumentError(
          "No stop sequences to check against. Did you forget to call AddStopTokenSequence()?");
    for (size_t item = 0; item < count; ++item) Step(lanes_[item], latest_tokens[item]);
    Publish();
    return OkStatus();
  }
  Status ProcessTokens(const std::vector<int>& latest_tokens) {
    return ProcessTokens(latest_tokens.data(), latest_tokens.size());
  }

  // Per item: length of the completed sequence plus the steps taken since (0 while still running).
  const std::vector<int>& GetStepsBeforeStopTokens() const { return steps_view_; }
  const std::vector<bool>& GetStopTokensFound() const { return stopped_view_; }

  StatusOr<bool> AllDone() const {
    if (lanes_.empty()) return FailedPreconditionError(
          "The Detector is not initialized with non-zero batch size. Did you forget to call ResetBatch() or "
          "AddStopTokenSequence() ??");
    for (const Lane& lane : lanes_)
      if (!lane.stopped) return false;
    return true;
  }

 private:
  struct Lane {
    std::vector<int> cursors;  // one per stop sequence
    int drop = 0;              // ids to drop from the end of this item's output
    bool stopped = false;
  };
  void Step(Lane& lane, int id) const {
    if (lane.stopped) {
      ++lane.drop;  // one more trailing step
      return;
    }
    // Every sequence sees the id, also after another one has completed on it: the last one to complete sets the count.
    for (size_t k = 0; k < sequences_.size(); ++k) {
      lane.cursors[k] = sequences_[k].Advance(lane.cursors[k], id);
      if (lane.cursors[k] == sequences_[k].length()) {
        lane.stopped = true;
        lane.drop = sequences_[k].length();
      }
    }
  }
  void Publish() {
    steps_view_.resize(lanes_.size());
    stopped_view_.resize(lanes_.size());
    for (size_t i = 0; i < lanes_.size(); ++i) {
      steps_view_[i] = lanes_[i].drop;
      stopped_view_[i] = lanes_[i].stopped;
    }
  }

  std::vector<StopSequence> sequences_;
  std::vector<Lane> lanes_;
  std::vector<int> steps_view_;     // what the two getters hand out by reference
  std::vector<bool> stopped_view_;
};

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_STOP_TOKEN_DETECTOR_H_
