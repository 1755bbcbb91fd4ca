#include "hip_llm_executor.h"

#include <algorithm>
#include <cstdio>
#include <utility>

namespace litert::lm {

StatusOr<std::unique_ptr<HipLlmExecutor>> HipLlmExecutor::Create(LlmExecutorSettings settings,
                                                                 std::unique_ptr<DecoderLayers> layers,
                                                                 HipExecutorOptions options,
                                                                 std::unique_ptr<AttentionBackend> backend) {
  if (!layers) return InvalidArgumentError("decoder layers must be provided.");
  if (settings.GetBackend() != Backend::GPU_HIP) return InvalidArgumentError("HipLlmExecutor needs Backend::GPU_HIP.");
  if (options.prefill_runner_lengths.empty()) return FailedPreconditionError("No prefill runner available.");
  for (int len : options.prefill_runner_lengths)
    if (len <= 0) return InvalidArgumentError("prefill runner lengths must be positive.");
  AttentionShape shape = layers->Shape();
  if (settings.GetMaxNumTokens() > 0) shape.max_tokens = settings.GetMaxNumTokens();
  if (shape.max_tokens <= 0) return InvalidArgumentError("max_num_tokens is not set.");
  settings.SetMaxNumTokens(shape.max_tokens);
  if (!backend) {
    const ActivationDataType act = settings.GetActivationDataType();
    if (act != ActivationDataType::FLOAT32 && act != ActivationDataType::FLOAT16)
      return UnimplementedError("HipLlmExecutor supports FLOAT32 and FLOAT16 activations.");
    ASSIGN_OR_RETURN(backend,
                     CreateMi355AttentionBackend(shape, act == ActivationDataType::FLOAT16, settings.GetDevice()));
  }
  return std::unique_ptr<HipLlmExecutor>(
      new HipLlmExecutor(std::move(settings), std::move(layers), std::move(options), std::move(backend)));
}

HipLlmExecutor::HipLlmExecutor(LlmExecutorSettings settings, std::unique_ptr<DecoderLayers> layers,
                               HipExecutorOptions options, std::unique_ptr<AttentionBackend> backend)
    : settings_(std::move(settings)),
      layers_(std::move(layers)),
      options_(std::move(options)),
      backend_(std::move(backend)) {
  for (int len : options_.prefill_runner_lengths) prefill_signature_map_[len] = "prefill_" + std::to_string(len);
  logits_ = TensorBuffer::Create(ElementType::kFloat32, {1, 1, layers_->VocabSize()});
}

Status HipLlmExecutor::Prefill(const ExecutorInputs& inputs, const ExecutorPrefillParams& params) {
  // The parameters are accepted and, like in the reference CPU executor, not
  // consulted: every attention call returns with its result in place.
  (void)params;
  ASSIGN_OR_RETURN(const TensorBuffer* ids_buffer, inputs.GetTextTokenIdsPtr());
  RET_CHECK_EQ(ids_buffer->dims().size(), 2u) << "Prefill token ids must be [batch, sequence_length].";
  // Only batch size 1 for now, as in the reference.
  RET_CHECK_EQ(ids_buffer->dims()[0], 1);
  RET_CHECK_GT(ids_buffer->dims()[1], 0) << "Prefill token ids must be non-empty.";
  RET_CHECK(ids_buffer->type() == ElementType::kInt32) << "Prefill token ids must be int32.";
  const int32_t* ids = ids_buffer->as<int32_t>();
  int remaining = ids_buffer->dims()[1];
  ASSIGN_OR_RETURN(auto work_groups, GetOptimizedPrefillWorkGroups(prefill_signature_map_, remaining));
  for (const auto& group : work_groups) {
    RETURN_IF_ERROR(PrefillInternal(ids, group.second));
    ids += group.second;
    remaining -= group.second;
  }
  RET_CHECK_EQ(remaining, 0).SetCode(StatusCode::kInternal) << "Work groups not covering the entire prefill input.";
  return OkStatus();
}

Status HipLlmExecutor::PrefillInternal(const int32_t* ids, int count) {
  // All ids but the last are executed now; a token left over from the previous
  // call goes first. The last id waits in next_input_token_id_ for the next
  // prefill or decode.
  std::vector<int32_t> tokens, positions;
  tokens.reserve(count);
  positions.reserve(count);
  const int limit = count - 1;
  if (limit == 0 && next_input_token_id_ != -1 && options_.execute_pending_on_single_id_chunk) {
    tokens.push_back(next_input_token_id_);
    positions.push_back(current_step_++);
    next_input_token_id_ = -1;
  }
  for (int i = 0; i < limit;) {
    if (next_input_token_id_ != -1) {
      tokens.push_back(next_input_token_id_);
      next_input_token_id_ = -1;
    } else {
      tokens.push_back(ids[i++]);
    }
    positions.push_back(current_step_++);
  }
  next_input_token_id_ = ids[count - 1];
  records_.push_back({false, tokens, positions});
  if (tokens.empty()) return OkStatus();
  return RunTokens(tokens, positions, /*is_decode=*/false, /*want_logits=*/false);
}

Status HipLlmExecutor::DecodeStep(const ExecutorInputs& inputs) {
  int id = next_input_token_id_;
  if (inputs.GetTextDataPtr().ok()) {
    const TensorBuffer& ids = (*inputs.GetTextDataPtr())->GetTokenIds();
    if (ids.HasValue() && ids.PackedSize() != 0) {
      // An explicit id wins over the pending one; one token, batch 1.
      RET_CHECK_EQ(ids.PackedSize(), sizeof(int32_t));
      id = ids.as<int32_t>()[0];
    }
  }
  if (id == -1) return InvalidArgumentError("No id available to be decoded.");
  next_input_token_id_ = -1;
  std::vector<int32_t> tokens{id}, positions{current_step_};
  records_.push_back({true, tokens, positions});
  RETURN_IF_ERROR(RunTokens(tokens, positions, /*is_decode=*/true, /*want_logits=*/true));
  ++current_step_;
  return OkStatus();
}

StatusOr<TensorBuffer> HipLlmExecutor::DecodeLogits(const ExecutorInputs& inputs) {
  RETURN_IF_ERROR(DecodeStep(inputs));
  return logits_.Duplicate();
}

Status HipLlmExecutor::Decode(const ExecutorInputs& inputs, TensorBuffer& output_logits) {
  RET_CHECK(output_logits.HasValue() && output_logits.type() == ElementType::kFloat32 &&
            output_logits.NumElements() == static_cast<size_t>(layers_->VocabSize()))
          .SetCode(StatusCode::kInvalidArgument)
      << "output_logits must be float32 [1, 1, vocab_size].";
  RETURN_IF_ERROR(DecodeStep(inputs));
  std::copy_n(logits_.as<float>(), layers_->VocabSize(), output_logits.as<float>());
  return OkStatus();
}

Status HipLlmExecutor::Decode(TensorBuffer& output_tokens) {
  RET_CHECK(output_tokens.HasValue() && output_tokens.type() == ElementType::kInt32 &&
            output_tokens.NumElements() >= 1)
          .SetCode(StatusCode::kInvalidArgument)
      << "output_tokens must be int32 [1, 1].";
  RETURN_IF_ERROR(DecodeStep(ExecutorInputs()));
  // Greedy pick, what the reference's built-in sampler (top-p with k = 1,
  // llm_litert_compiled_model_executor.cc:548-553) reduces to.
  const float* logits = logits_.as<float>();
  const int vocab = layers_->VocabSize();
  int best = static_cast<int>(std::max_element(logits, logits + vocab) - logits);
  if (best < 0) {
    std::fprintf(stderr, "Invalid decode and sample result. The sampled token is casted to 0 to avoid crash.\n");
    best = 0;
  }
  output_tokens.as<int32_t>()[0] = best;
  next_input_token_id_ = best;
  return OkStatus();
}

Status HipLlmExecutor::Reset() {
  // Steps and the pending token are forgotten; the cache memory is left as it
  // is, stale rows can never be seen again because visibility ends at the
  // current step (llm_litert_compiled_model_executor.cc:568-574).
  current_step_ = 0;
  next_input_token_id_ = -1;
  records_.clear();
  return backend_->Reset();
}

Status HipLlmExecutor::RunTokens(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions,
                                 bool is_decode, bool want_logits) {
  const AttentionShape& shape = layers_->Shape();
  const int n = static_cast<int>(tokens.size());
  const int pos0 = positions.front();
  if (pos0 + n > settings_.GetMaxNumTokens())
    return OutOfRangeError("KV cache is full: step " + std::to_string(pos0 + n) + " exceeds max_num_tokens " +
                           std::to_string(settings_.GetMaxNumTokens()) + ".");
  const size_t qn = static_cast<size_t>(n) * shape.num_q_heads * shape.head_dim;
  const size_t kn = static_cast<size_t>(n) * shape.num_kv_heads * shape.head_dim;
  q_.resize(qn);
  attn_.resize(qn);
  k_.resize(kn);
  v_.resize(kn);
  RETURN_IF_ERROR(layers_->Begin(tokens, positions));
  for (int layer = 0; layer < shape.num_layers; ++layer) {
    RETURN_IF_ERROR(layers_->ProjectQkv(layer, q_.data(), k_.data(), v_.data()));
    if (shape.transforms.empty()) {
      RETURN_IF_ERROR(backend_->Append(layer, pos0, n, k_.data(), v_.data()));
    } else {
      // raw projections: norm + rotary embedding + cache write in one device pass
      RETURN_IF_ERROR(backend_->PreAttention(layer, pos0, n, q_.data(), k_.data(), v_.data()));
    }
    if (is_decode) {
      RETURN_IF_ERROR(backend_->Decode(layer, pos0 + 1, q_.data(), attn_.data()));
    } else {
      RETURN_IF_ERROR(backend_->Prefill(layer, pos0, n, q_.data(), attn_.data()));
    }
    RETURN_IF_ERROR(layers_->ConsumeAttention(layer, attn_.data()));
  }
  if (want_logits) RETURN_IF_ERROR(layers_->Logits(logits_.as<float>()));
  return OkStatus();
}

}  // namespace litert::lm
