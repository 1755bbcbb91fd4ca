#include "hip_llm_executor.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <utility>

#include "../../include/mi355_sampler.h"

namespace litert::lm {
namespace {
Status HipStatus(hipError_t e, const char* what) {
  if (e == hipSuccess) return OkStatus();
  return InternalError(std::string(what) + ": " + hipGetErrorString(e));
}
Status SamplerStatus(int rc, char* err, const char* what) {
  if (rc == MI355_SAMPLER_OK) return OkStatus();
  std::string msg = std::string(what) + ": " + (err ? err : "(no message)");
  free(err);
  return Status(static_cast<StatusCode>(rc), msg);
}
}  // namespace

// Everything the device-resident mode keeps in device memory between calls.
struct HipLlmExecutor::DeviceState {
  int device = 0;
  bool fp16 = false;
  DecoderLayers::DeviceActivations io;  // q / k / v / attention output of one pass, sized for `capacity` tokens
  int capacity = 0;
  float* logits = nullptr;       // [vocab] float32
  int32_t* sampled = nullptr;    // [1]
  int32_t* host_id = nullptr;    // pinned, the one value that returns per decode step
  mi355_sampler* sampler = nullptr;
  bool logits_fetched = false;   // logits_ (host) holds the logits of the last step

  ~DeviceState() {
    (void)hipSetDevice(device);
    if (sampler) mi355_sampler_destroy(sampler);
    for (void* p : {io.q, io.k, io.v, io.attn, static_cast<void*>(logits), static_cast<void*>(sampled)})
      if (p) (void)hipFree(p);
    if (host_id) (void)hipHostFree(host_id);
  }
};

HipLlmExecutor::~HipLlmExecutor() {
  // queued passes still read the buffers: drain before the members go away
  if (device_) (void)backend_->Sync();
}

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
  using Residency = HipExecutorOptions::Residency;
  const ActivationDataType act = settings.GetActivationDataType();
  bool on_device;
  if (!backend) {
    if (act != ActivationDataType::FLOAT32 && act != ActivationDataType::FLOAT16)
      return UnimplementedError("HipLlmExecutor supports FLOAT32 and FLOAT16 activations.");
    on_device = options.residency == Residency::kDevice ||
                (options.residency == Residency::kAuto && layers->HasDeviceForm());
    if (on_device && !layers->HasDeviceForm())
      return InvalidArgumentError("device-resident execution needs decoder layers with a device form.");
    ASSIGN_OR_RETURN(backend, CreateMi355AttentionBackend(shape, act == ActivationDataType::FLOAT16,
                                                          settings.GetDevice(), on_device));
  } else {
    on_device = backend->DeviceResident();
    if (options.residency == Residency::kDevice && !on_device)
      return InvalidArgumentError("device-resident execution needs a device-resident attention backend.");
    if (options.residency == Residency::kHost && on_device)
      return InvalidArgumentError("host-staged execution needs a host-staged attention backend.");
    if (on_device && !layers->HasDeviceForm())
      return InvalidArgumentError("device-resident execution needs decoder layers with a device form.");
  }
  std::unique_ptr<HipLlmExecutor> ex(
      new HipLlmExecutor(std::move(settings), std::move(layers), std::move(options), std::move(backend)));
  if (on_device) RETURN_IF_ERROR(ex->InitDeviceState());
  return ex;
}

Status HipLlmExecutor::InitDeviceState() {
  auto st = std::make_unique<DeviceState>();
  st->device = settings_.GetDevice();
  st->fp16 = settings_.GetActivationDataType() == ActivationDataType::FLOAT16;
  st->io.fp16 = st->fp16;
  st->io.stream = backend_->Stream();
  RETURN_IF_ERROR(HipStatus(hipSetDevice(st->device), "hipSetDevice"));
  const AttentionShape& shape = layers_->Shape();
  // One pass never holds more tokens than the longest prefill runner.
  int capacity = 1;
  for (int len : options_.prefill_runner_lengths) capacity = std::max(capacity, len);
  const size_t esz = st->fp16 ? 2 : 4;
  const size_t qn = (size_t)capacity * shape.num_q_heads * shape.head_dim * esz;
  const size_t kn = (size_t)capacity * shape.num_kv_heads * shape.head_dim * esz;
  RETURN_IF_ERROR(HipStatus(hipMalloc(&st->io.q, qn), "hipMalloc(q)"));
  RETURN_IF_ERROR(HipStatus(hipMalloc(&st->io.attn, qn), "hipMalloc(attn)"));
  RETURN_IF_ERROR(HipStatus(hipMalloc(&st->io.k, kn), "hipMalloc(k)"));
  RETURN_IF_ERROR(HipStatus(hipMalloc(&st->io.v, kn), "hipMalloc(v)"));
  RETURN_IF_ERROR(HipStatus(hipMalloc(&st->logits, sizeof(float) * (size_t)layers_->VocabSize()), "hipMalloc(logits)"));
  RETURN_IF_ERROR(HipStatus(hipMalloc(&st->sampled, sizeof(int32_t)), "hipMalloc(id)"));
  RETURN_IF_ERROR(HipStatus(hipHostMalloc(&st->host_id, sizeof(int32_t)), "hipHostMalloc(id)"));
  st->capacity = capacity;
  device_ = std::move(st);
  return OkStatus();
}

Status HipLlmExecutor::WaitForCompletion() { return device_ ? backend_->Sync() : OkStatus(); }

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
  // wait_for_completion: host-staged passes have completed when they return; device-resident passes are only
  // queued, and the call waits for them when asked to. The cancel flag is looked at before every chunk: chunks
  // already run stay run (their rows are in the cache and counted in the step), the rest is dropped.
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
    if (params.GetCancelFlag() != nullptr && params.GetCancelFlag()->load(std::memory_order_relaxed))
      return CancelledError("Prefill was cancelled.");
    RETURN_IF_ERROR(PrefillInternal(ids, group.second));
    ids += group.second;
    remaining -= group.second;
  }
  RET_CHECK_EQ(remaining, 0).SetCode(StatusCode::kInternal) << "Work groups not covering the entire prefill input.";
  if (params.GetWaitForCompletion()) RETURN_IF_ERROR(WaitForCompletion());
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

Status HipLlmExecutor::FetchLogits() {
  if (!device_ || device_->logits_fetched) return OkStatus();
  hipStream_t stream = static_cast<hipStream_t>(device_->io.stream);
  RETURN_IF_ERROR(HipStatus(hipMemcpyAsync(logits_.as<float>(), device_->logits, logits_.PackedSize(),
                                           hipMemcpyDeviceToHost, stream),
                            "hipMemcpyAsync(logits)"));
  RETURN_IF_ERROR(backend_->Sync());  // the logits buffer handed out is host-visible
  device_->logits_fetched = true;
  return OkStatus();
}

StatusOr<TensorBuffer> HipLlmExecutor::DecodeLogits(const ExecutorInputs& inputs) {
  RETURN_IF_ERROR(DecodeStep(inputs));
  RETURN_IF_ERROR(FetchLogits());
  return logits_.Duplicate();
}

Status HipLlmExecutor::Decode(const ExecutorInputs& inputs, TensorBuffer& output_logits) {
  RET_CHECK(output_logits.HasValue() && output_logits.type() == ElementType::kFloat32 &&
            output_logits.NumElements() == static_cast<size_t>(layers_->VocabSize()))
          .SetCode(StatusCode::kInvalidArgument)
      << "output_logits must be float32 [1, 1, vocab_size].";
  RETURN_IF_ERROR(DecodeStep(inputs));
  RETURN_IF_ERROR(FetchLogits());
  std::copy_n(logits_.as<float>(), layers_->VocabSize(), output_logits.as<float>());
  return OkStatus();
}

Status HipLlmExecutor::Decode(TensorBuffer& output_tokens) {
  RET_CHECK(output_tokens.HasValue() && output_tokens.type() == ElementType::kInt32 &&
            output_tokens.NumElements() >= 1)
          .SetCode(StatusCode::kInvalidArgument)
      << "output_tokens must be int32 [1, 1].";
  RETURN_IF_ERROR(DecodeStep(ExecutorInputs()));
  const int vocab = layers_->VocabSize();
  int best;
  if (device_) {
    // The reference's built-in sampler: top-p with k = 1, p = 0, temperature 1, seed 0, made on first use and
    // dropped by Reset (llm_litert_compiled_model_executor.cc:536-566). It runs on the stream of the pass, reads
    // the logits where they are and only the id crosses to the host.
    if (!device_->sampler) {
      mi355_sampler_config cfg{};
      cfg.struct_size = sizeof(cfg);
      cfg.batch_size = 1;
      cfg.vocab_size = vocab;
      cfg.type = MI355_SAMPLER_TOP_P;
      cfg.k = 1;
      cfg.p = 0.0f;
      cfg.temperature = 1.0f;
      cfg.seed = 0;
      cfg.device = device_->device;
      cfg.host_io = 0;
      cfg.own_stream = 0;
      cfg.stream = device_->io.stream;
      char* err = nullptr;
      const int rc = mi355_sampler_create(&cfg, &device_->sampler, &err);
      RETURN_IF_ERROR(SamplerStatus(rc, err, "mi355_sampler_create"));
    }
    char* err = nullptr;
    const int rc = mi355_sampler_sample(device_->sampler, device_->logits, device_->sampled, nullptr, &err);
    RETURN_IF_ERROR(SamplerStatus(rc, err, "mi355_sampler_sample"));
    RETURN_IF_ERROR(HipStatus(hipMemcpyAsync(device_->host_id, device_->sampled, sizeof(int32_t), hipMemcpyDeviceToHost,
                                             static_cast<hipStream_t>(device_->io.stream)),
                              "hipMemcpyAsync(id)"));
    RETURN_IF_ERROR(backend_->Sync());  // output_tokens is host-visible
    best = *device_->host_id;
  } else {
    // Greedy pick, what that sampler reduces to.
    const float* logits = logits_.as<float>();
    best = static_cast<int>(std::max_element(logits, logits + vocab) - logits);
  }
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
  if (device_) {
    RETURN_IF_ERROR(backend_->Sync());
    if (device_->sampler) mi355_sampler_destroy(device_->sampler);
    device_->sampler = nullptr;
    device_->logits_fetched = false;
  }
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
  if (device_) return RunTokensOnDevice(tokens, positions, is_decode, want_logits);
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

// The same pass with every buffer in device memory and nothing waited for: the layers and the attention calls are
// queued on the backend's stream in dependency order.
Status HipLlmExecutor::RunTokensOnDevice(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions,
                                         bool is_decode, bool want_logits) {
  const AttentionShape& shape = layers_->Shape();
  const int n = static_cast<int>(tokens.size());
  const int pos0 = positions.front();
  RET_CHECK_LE(n, device_->capacity) << "a pass of " << n << " tokens exceeds the longest prefill runner.";
  RETURN_IF_ERROR(HipStatus(hipSetDevice(device_->device), "hipSetDevice"));
  const DecoderLayers::DeviceActivations& io = device_->io;
  RETURN_IF_ERROR(layers_->BeginOnDevice(tokens, positions, io));
  // One-token passes over layers with a transform: the step before attention and the attention in one launch.
  const bool single_call_step = options_.single_call_decode_step && is_decode && n == 1 && !shape.transforms.empty() &&
                                backend_->HasDecodeStep();
  for (int layer = 0; layer < shape.num_layers; ++layer) {
    if (single_call_step) {
      RETURN_IF_ERROR(backend_->DecodeStepOnDevice(layer, pos0 + 1, io.q, io.k, io.v, io.attn));
      RETURN_IF_ERROR(layers_->NextLayerOnDevice(layer, io));
      continue;
    }
    if (shape.transforms.empty()) {
      RETURN_IF_ERROR(backend_->AppendOnDevice(layer, pos0, n, io.k, io.v));
    } else {
      RETURN_IF_ERROR(backend_->PreAttentionOnDevice(layer, pos0, n, io.q, io.k, io.v));
    }
    if (is_decode) {
      RETURN_IF_ERROR(backend_->DecodeOnDevice(layer, pos0 + 1, io.q, io.attn));
    } else {
      RETURN_IF_ERROR(backend_->PrefillOnDevice(layer, pos0, n, io.q, io.attn));
    }
    RETURN_IF_ERROR(layers_->NextLayerOnDevice(layer, io));
  }
  if (want_logits) {
    RETURN_IF_ERROR(layers_->LogitsOnDevice(device_->logits, io.stream));
    device_->logits_fetched = false;
  }
  return OkStatus();
}

}  // namespace litert::lm
