// The loop above the executor that the reference's benchmark protocol runs
// (runtime/core/pipeline.cc:231-367): one Prefill turn over the prompt ids, then
// Decode steps with sampling inside the executor until a stop sequence, the
// requested number of benchmark steps or the KV-cache limit ends them - with
// the turns timed into a BenchmarkInfo when one is given. Tokenisation is not
// part of this build: prompts arrive and responses leave as token ids.
#ifndef LITERT_LM_AMD_EXECUTOR_PIPELINE_H_
#define LITERT_LM_AMD_EXECUTOR_PIPELINE_H_

#include <functional>
#include <optional>
#include <vector>

#include "benchmark_info.h"
#include "llm_executor_base.h"
#include "stop_token_detector.h"

namespace litert::lm {

// Prefills `prompt_ids` (bos_token_id is put in front, as the reference does
// after tokenising). With a benchmark that names a prefill token count the ids
// are resized to exactly that many (padded with 0 / cut) and no bos is added.
// kInvalidArgument when the ids do not leave room in max_num_tokens.
// Returns the last prefilled id. pipeline.cc:231-276.
StatusOr<int> Prefill(LlmExecutor& executor, std::vector<int> prompt_ids, int bos_token_id, bool wait_for_completion,
                      std::optional<BenchmarkInfo>& benchmark_info);

// Decodes until ShouldStop (pipeline.cc:64-84): a stop sequence (only when no
// benchmark step count is set), the benchmark's step count, or current_step >=
// max_num_tokens. Returns every id produced, the stop tokens included.
// pipeline.cc:278-318.
StatusOr<std::vector<int>> Decode(LlmExecutor& executor, const StopTokenDetector& stop_token_detector,
                                  std::optional<BenchmarkInfo>& benchmark_info);

// The same with each id handed to `on_next` as it is produced; when the cache
// limit ends the loop `on_error` receives kInternal "Maximum kv-cache size
// reached." first. pipeline.cc:320-367.
Status DecodeStreaming(LlmExecutor& executor, const StopTokenDetector& stop_token_detector,
                       std::optional<BenchmarkInfo>& benchmark_info, const std::function<void(int)>& on_next,
                       const std::function<void(const Status&)>& on_error);

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_PIPELINE_H_
