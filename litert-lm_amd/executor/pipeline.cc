#include "pipeline.h"

#include <string>
#include <utility>

namespace litert::lm {
namespace {

// Why a decode loop ends (runtime/core/pipeline.cc:64-84), in the order the conditions are tried.
enum class LoopEnd { kGoOn, kStopTokens, kStepBudget, kCacheFull };

struct LoopLimits {
  int forced_steps;    // benchmark's decode step count, 0 = none: then a stop sequence ends the loop
  int max_num_tokens;  // KV-cache capacity in steps
};

LoopLimits LimitsOf(const LlmExecutor& executor, const std::optional<BenchmarkInfo>& benchmark_info) {
  // An executor that cannot report its settings is taken to hold 4096 tokens (pipeline.cc:50-62).
  auto settings = executor.GetExecutorSettings();
  return LoopLimits{benchmark_info.has_value() ? benchmark_info->GetBenchmarkParams().num_decode_tokens : 0,
                    settings.ok() ? settings->GetMaxNumTokens() : 4096};
}

LoopEnd Judge(const LoopLimits& limits, bool stop_tokens_seen, int steps_done, int current_step) {
  if (limits.forced_steps == 0 && stop_tokens_seen) return LoopEnd::kStopTokens;
  if (limits.forced_steps > 0 && steps_done >= limits.forced_steps) return LoopEnd::kStepBudget;
  if (current_step >= limits.max_num_tokens) return LoopEnd::kCacheFull;
  return LoopEnd::kGoOn;
}

// The loop both decode entry points share. Each step: Decode(tokens) with sampling inside the executor, timed as
// the mark "executor_decode_and_sample" (pipeline.cc:160-227), the id shown to the stop detector (a private copy:
// the caller's keeps its state) and to `emit`; `on_cache_full`, when given, hears of the cache limit before the
// loop ends. A failed step is returned as it is, after `on_failure` (when given) has seen it.
Status RunDecodeLoop(LlmExecutor& executor, StopTokenDetector detector, std::optional<BenchmarkInfo>& benchmark_info,
                     const std::function<void(int)>& emit, const std::function<void(const Status&)>& on_failure,
                     const std::function<void(const Status&)>& on_cache_full) {
  static const char kMark[] = "executor_decode_and_sample";
  const LoopLimits limits = LimitsOf(executor, benchmark_info);
  if (benchmark_info.has_value()) RETURN_IF_ERROR(benchmark_info->TimeDecodeTurnStart());
  TensorBuffer id_buffer = TensorBuffer::Create(ElementType::kInt32, {1, 1});
  auto step = [&]() -> StatusOr<bool> {
    if (benchmark_info.has_value()) RETURN_IF_ERROR(benchmark_info->TimeMarkDelta(kMark));
    RETURN_IF_ERROR(executor.Decode(id_buffer));
    if (benchmark_info.has_value()) RETURN_IF_ERROR(benchmark_info->TimeMarkDelta(kMark));
    if (id_buffer.NumElements() != 1) return InternalError("Unexpected number of decoded tokens.");
    RETURN_IF_ERROR(detector.ProcessTokens(id_buffer.as<int32_t>(), 1));
    return detector.AllDone();
  };
  int steps_done = 0;
  for (LoopEnd end = LoopEnd::kGoOn; end == LoopEnd::kGoOn;) {
    const StatusOr<bool> stop_tokens_seen = step();
    if (!stop_tokens_seen.ok()) {
      if (on_failure) on_failure(stop_tokens_seen.status());
      return stop_tokens_seen.status();
    }
    ++steps_done;
    if (emit) emit(id_buffer.as<int32_t>()[0]);
    ASSIGN_OR_RETURN(const int current_step, executor.GetCurrentStep());
    end = Judge(limits, *stop_tokens_seen, steps_done, current_step);
    if (end == LoopEnd::kCacheFull && on_cache_full) on_cache_full(InternalError("Maximum kv-cache size reached."));
  }
  if (benchmark_info.has_value()) RETURN_IF_ERROR(benchmark_info->TimeDecodeTurnEnd(steps_done));
  return OkStatus();
}

}  // namespace

StatusOr<int> Prefill(LlmExecutor& executor, std::vector<int> ids, int bos_token_id, bool wait_for_completion,
                      std::optional<BenchmarkInfo>& benchmark_info) {
  // A benchmark that names a prefill length decides the ids' count (cut, or padded with 0); otherwise the
  // begin-of-sequence id goes in front (pipeline.cc:231-252).
  const int forced = benchmark_info.has_value() ? benchmark_info->GetBenchmarkParams().num_prefill_tokens : 0;
  if (benchmark_info.has_value()) RETURN_IF_ERROR(benchmark_info->TimePrefillTurnStart());
  if (forced > 0) ids.resize(forced);
  else ids.insert(ids.begin(), bos_token_id);

  auto settings = executor.GetExecutorSettings();
  const int max_num_tokens = settings.ok() ? settings->GetMaxNumTokens() : 4096;
  const int count = static_cast<int>(ids.size());
  if (count >= max_num_tokens)
    return InvalidArgumentError("Input token ids are too long. Exceeding the maximum number of tokens allowed: " +
                                std::to_string(count) + " >= " + std::to_string(max_num_tokens));
  if (count == 0) return InternalError("Input token ids are empty.");

  ExecutorPrefillParams params;
  params.SetWaitForCompletion(wait_for_completion);
  ExecutorInputs inputs(ExecutorTextData(TensorBuffer::CopyFrom(ElementType::kInt32, {1, count}, ids.data())));
  RETURN_IF_ERROR(executor.Prefill(inputs, params));
  if (benchmark_info.has_value()) RETURN_IF_ERROR(benchmark_info->TimePrefillTurnEnd(count));
  return ids.back();
}

Status DecodeStreaming(LlmExecutor& executor, const StopTokenDetector& stop_token_detector,
                       std::optional<BenchmarkInfo>& benchmark_info, const std::function<void(int)>& on_next,
                       const std::function<void(const Status&)>& on_error) {
  // The observer hears of failed steps and of the cache limit (pipeline.cc:320-367).
  return RunDecodeLoop(executor, stop_token_detector, benchmark_info, on_next, on_error, on_error);
}

StatusOr<std::vector<int>> Decode(LlmExecutor& executor, const StopTokenDetector& stop_token_detector,
                                  std::optional<BenchmarkInfo>& benchmark_info) {
  // No observer: the cache limit ends the loop silently (pipeline.cc:278-318).
  std::vector<int> ids;
  RETURN_IF_ERROR(RunDecodeLoop(executor, stop_token_detector, benchmark_info, [&ids](int id) { ids.push_back(id); },
                                nullptr, nullptr));
  return ids;
}

}  // namespace litert::lm
