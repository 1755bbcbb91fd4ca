// C test surface of HipLlmExecutor for the Python tests (ctypes): create an
// executor over the synthetic decoder layers, drive Prefill / Decode, read the
// trace of forward passes. Status codes are absl::StatusCode integers; error
// text is malloc'd for the caller to free().
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <memory>

#include <sstream>

#include "benchmark_info.h"
#include "fake_llm_executor.h"
#include "hip_llm_executor.h"
#include "litertlm_reader.h"
#include "model_file.h"
#include "pipeline.h"
#include "stop_token_detector.h"

using namespace litert::lm;

namespace {
int Finish(const Status& s, char** err) {
  if (!s.ok() && err) {
    *err = static_cast<char*>(malloc(s.message().size() + 1));
    if (*err) memcpy(*err, s.message().c_str(), s.message().size() + 1);
  }
  return static_cast<int>(s.code());
}
ExecutorInputs IdsInput(const int32_t* ids, int batch, int n) {
  return ExecutorInputs(ExecutorTextData(TensorBuffer::CopyFrom(ElementType::kInt32, {batch, n}, ids)));
}
char* CopyText(const std::string& text) {
  char* out = static_cast<char*>(malloc(text.size() + 1));
  if (out) memcpy(out, text.c_str(), text.size() + 1);
  return out;
}
}  // namespace

extern "C" {

struct hle_config {
  int32_t num_layers, num_q_heads, num_kv_heads, vocab, max_num_tokens;
  const int32_t* layer_window;       // [num_layers] or null
  const int32_t* runner_lengths;     // [num_runners]
  int32_t num_runners;
  int32_t fp16_activations;          // 0: float32, 1: float16
  int32_t recording_backend;         // 1: no GPU, attention returns zeros and records calls
  int32_t execute_pending_on_single_id_chunk;
  float softcap;
  int32_t pre_attention;             // 1: the layers hand over raw projections; Gemma-3-like norm + rotary constants
  int32_t device_resident;           // -1: the executor decides, 0: host-staged, 1: device-resident
  int32_t two_call_decode_step;      // 1: device-resident decode keeps pre-attention and attention as two calls per layer
};

int hle_create(const hle_config* c, void** out, char** err) {
  *out = nullptr;
  AttentionShape shape;
  shape.num_layers = c->num_layers;
  shape.num_q_heads = c->num_q_heads;
  shape.num_kv_heads = c->num_kv_heads;
  shape.head_dim = 256;
  shape.max_tokens = c->max_num_tokens;
  shape.softcap = c->softcap;
  if (c->layer_window) shape.layer_window.assign(c->layer_window, c->layer_window + c->num_layers);
  if (c->pre_attention) shape.transforms = SyntheticDecoderLayers::Transforms(shape);
  auto settings = LlmExecutorSettings::CreateDefault(Backend::GPU_HIP);
  if (!settings.ok()) return Finish(settings.status(), err);
  settings->SetMaxNumTokens(c->max_num_tokens);
  settings->SetActivationDataType(c->fp16_activations ? ActivationDataType::FLOAT16 : ActivationDataType::FLOAT32);
  HipExecutorOptions options;
  options.prefill_runner_lengths.assign(c->runner_lengths, c->runner_lengths + c->num_runners);
  options.execute_pending_on_single_id_chunk = c->execute_pending_on_single_id_chunk != 0;
  options.residency = c->device_resident < 0    ? HipExecutorOptions::Residency::kAuto
                      : c->device_resident == 0 ? HipExecutorOptions::Residency::kHost
                                                : HipExecutorOptions::Residency::kDevice;
  options.single_call_decode_step = c->two_call_decode_step == 0;
  std::unique_ptr<AttentionBackend> backend;
  if (c->recording_backend) backend = std::make_unique<RecordingAttentionBackend>(shape);
  auto ex = HipLlmExecutor::Create(*settings, std::make_unique<SyntheticDecoderLayers>(shape, c->vocab), options,
                                   std::move(backend));
  if (!ex.ok()) return Finish(ex.status(), err);
  *out = ex->release();
  return 0;
}

void hle_destroy(void* h) { delete static_cast<HipLlmExecutor*>(h); }

int hle_prefill(void* h, const int32_t* ids, int32_t batch, int32_t n, char** err) {
  return Finish(static_cast<HipLlmExecutor*>(h)->Prefill(IdsInput(ids, batch, n)), err);
}

// Prefill with parameters: `cancel` is the value the caller's cancel flag holds during the call (-1: no flag).
int hle_prefill_with_params(void* h, const int32_t* ids, int32_t batch, int32_t n, int32_t wait_for_completion,
                            int32_t cancel, char** err) {
  std::atomic_bool flag(cancel > 0);
  ExecutorPrefillParams params(-1, wait_for_completion != 0, cancel < 0 ? nullptr : &flag);
  return Finish(static_cast<HipLlmExecutor*>(h)->Prefill(IdsInput(ids, batch, n), params), err);
}
int hle_is_device_resident(void* h) { return static_cast<HipLlmExecutor*>(h)->device_resident() ? 1 : 0; }
int hle_wait_for_completion(void* h, char** err) {
  return Finish(static_cast<HipLlmExecutor*>(h)->WaitForCompletion(), err);
}

int hle_decode(void* h, int32_t* out_token, char** err) {
  TensorBuffer out = TensorBuffer::Create(ElementType::kInt32, {1, 1});
  Status s = static_cast<HipLlmExecutor*>(h)->Decode(out);
  if (s.ok()) *out_token = out.as<int32_t>()[0];
  return Finish(s, err);
}

// explicit_id < 0: use the pending token.
int hle_decode_logits(void* h, int32_t explicit_id, float* logits, char** err) {
  auto* ex = static_cast<HipLlmExecutor*>(h);
  ExecutorInputs inputs = explicit_id >= 0 ? IdsInput(&explicit_id, 1, 1) : ExecutorInputs();
  auto r = ex->DecodeLogits(inputs);
  if (!r.ok()) return Finish(r.status(), err);
  memcpy(logits, r->as<float>(), r->PackedSize());
  return 0;
}

int hle_current_step(void* h) { return *static_cast<HipLlmExecutor*>(h)->GetCurrentStep(); }
int hle_vocab_size(void* h) { return *static_cast<HipLlmExecutor*>(h)->GetVocabSize(); }
int hle_max_num_tokens(void* h) { return static_cast<HipLlmExecutor*>(h)->GetExecutorSettings()->GetMaxNumTokens(); }
int hle_reset(void* h, char** err) { return Finish(static_cast<HipLlmExecutor*>(h)->Reset(), err); }
// The base class's default: no vision input in this executor.
int hle_fill_vision_embeddings(void* h, int32_t image_index, char** err) {
  return Finish(static_cast<HipLlmExecutor*>(h)->FillVisionEmbeddings(ExecutorVisionData(), image_index), err);
}
const char* hle_backend_name(void* h) {
  static thread_local std::string name;
  name = std::string(static_cast<HipLlmExecutor*>(h)->ExecutorBackendName());
  return name.c_str();
}

int hle_num_runs(void* h) { return static_cast<int>(static_cast<HipLlmExecutor*>(h)->run_records().size()); }
// Copies run `i`: returns its token count; is_decode, tokens and positions are filled (capacity `cap`).
int hle_get_run(void* h, int i, int32_t* is_decode, int32_t* tokens, int32_t* positions, int cap) {
  const auto& r = static_cast<HipLlmExecutor*>(h)->run_records()[i];
  *is_decode = r.is_decode ? 1 : 0;
  const int n = static_cast<int>(r.tokens.size());
  for (int j = 0; j < n && j < cap; ++j) {
    tokens[j] = r.tokens[j];
    positions[j] = r.positions[j];
  }
  return n;
}

int hle_backend_from_string(const char* s) {
  auto b = GetBackendFromString(s);
  return b.ok() ? static_cast<int>(*b) : -static_cast<int>(b.status().code());
}

// Chunk plan for `n` ids over the given runner lengths: fills lens[] with the
// runner length and counts[] with the ids of each call; returns the number of calls.
int hle_plan(const int32_t* runner_lengths, int num_runners, int n, int32_t* lens, int32_t* counts, int cap) {
  SortedPrefillSignatureMap m;
  for (int i = 0; i < num_runners; ++i) m[runner_lengths[i]] = std::to_string(runner_lengths[i]);
  auto g = GetOptimizedPrefillWorkGroups(m, n);
  if (!g.ok()) return -static_cast<int>(g.status().code());
  int k = 0;
  for (const auto& e : *g) {
    if (k < cap) {
      lens[k] = std::stoi(e.first);
      counts[k] = e.second;
    }
    ++k;
  }
  return k;
}

// ---- BenchmarkInfo, stop-token detector and the prefill / decode loop (test surface)

void* hle_bi_create(int32_t num_prefill_tokens, int32_t num_decode_tokens) {
  BenchmarkParams p;
  p.num_prefill_tokens = num_prefill_tokens;
  p.num_decode_tokens = num_decode_tokens;
  return new BenchmarkInfo(p);
}
void hle_bi_destroy(void* bi) { delete static_cast<BenchmarkInfo*>(bi); }

// what: 0/1 init phase start/end, 2/3 prefill turn start/end, 4/5 decode turn start/end, 6 mark
int hle_bi_call(void* bi, int32_t what, const char* name, uint64_t tokens, char** err) {
  auto* b = static_cast<BenchmarkInfo*>(bi);
  switch (what) {
    case 0: return Finish(b->TimeInitPhaseStart(name), err);
    case 1: return Finish(b->TimeInitPhaseEnd(name), err);
    case 2: return Finish(b->TimePrefillTurnStart(), err);
    case 3: return Finish(b->TimePrefillTurnEnd(tokens), err);
    case 4: return Finish(b->TimeDecodeTurnStart(), err);
    case 5: return Finish(b->TimeDecodeTurnEnd(tokens), err);
    case 6: return Finish(b->TimeMarkDelta(name), err);
    default: return Finish(InvalidArgumentError("unknown call"), err);
  }
}
// what: 0 init phases, 1 prefill turns, 2 decode turns, 3 marks
int hle_bi_count(void* bi, int32_t what) {
  auto* b = static_cast<BenchmarkInfo*>(bi);
  switch (what) {
    case 0: return static_cast<int>(b->GetInitPhases().size());
    case 1: return static_cast<int>(b->GetTotalPrefillTurns());
    case 2: return static_cast<int>(b->GetTotalDecodeTurns());
    default: return static_cast<int>(b->GetMarkDurations().size());
  }
}
// Seconds of an init phase (what 0) or mark (what 3) by name, tokens per second of a prefill (1) / decode (2) turn by index; -1 if absent.
double hle_bi_value(void* bi, int32_t what, const char* name, int32_t index) {
  auto* b = static_cast<BenchmarkInfo*>(bi);
  if (what == 1) return b->GetPrefillTokensPerSec(index);
  if (what == 2) return b->GetDecodeTokensPerSec(index);
  const auto& m = what == 0 ? b->GetInitPhases() : b->GetMarkDurations();
  auto it = m.find(name);
  return it == m.end() ? -1.0 : static_cast<double>(it->second.count()) * 1e-9;
}
char* hle_bi_report(void* bi) {
  std::ostringstream os;
  os << *static_cast<BenchmarkInfo*>(bi);
  return CopyText(os.str());
}
char* hle_format_duration(int64_t ns) { return CopyText(FormatDuration(Duration(ns))); }

// Feeds tokens [steps][batch] step by step until every item has stopped; returns the index of that step (steps if
// never). add_codes[n_seqs] receives the status of each AddStopTokenSequence, steps_before[batch] the detector's
// count per item; reset != 0 calls ResetBatch() at the end and reports AllDone after it in *done_after_reset.
int hle_stop_detector_run(int32_t batch, const int32_t* seqs_flat, const int32_t* seq_lens, int32_t n_seqs,
                          const int32_t* tokens, int32_t steps, int32_t* add_codes, int32_t* steps_before,
                          int32_t reset, int32_t* done_after_reset) {
  StopTokenDetector detector(batch);
  const int32_t* p = seqs_flat;
  for (int i = 0; i < n_seqs; ++i) {
    add_codes[i] = static_cast<int>(detector.AddStopTokenSequence(std::vector<int>(p, p + seq_lens[i])).code());
    p += seq_lens[i];
  }
  int i = 0;
  for (; i < steps; ++i) {
    Status s = detector.ProcessTokens(tokens + (size_t)i * batch, batch);
    if (!s.ok()) return -static_cast<int>(s.code());
    if (*detector.AllDone()) break;
  }
  if (reset) {
    detector.ResetBatch();
    *done_after_reset = *detector.AllDone() ? 1 : 0;
  }
  for (int b = 0; b < batch; ++b) steps_before[b] = detector.GetStepsBeforeStopTokens()[b];
  return i;
}

struct hle_loop_result {
  int32_t last_prefill_id;
  int32_t n_tokens;          // ids produced by the decode loop
  int32_t cache_full_error;  // the streaming observer saw "Maximum kv-cache size reached."
  int32_t current_step;
};

namespace {
int RunLoop(LlmExecutor& ex, const int32_t* prompt, int n_prompt, int bos, const int32_t* stop_seq, int n_stop,
            int bench_prefill, int bench_decode, int streaming, int do_prefill, int32_t* out_tokens, int cap,
            hle_loop_result* res, char** report, char** err) {
  std::optional<BenchmarkInfo> info;
  if (bench_prefill > 0 || bench_decode > 0) {
    BenchmarkParams p;
    p.num_prefill_tokens = bench_prefill;
    p.num_decode_tokens = bench_decode;
    info.emplace(p);
  }
  *res = hle_loop_result{-1, 0, 0, 0};
  if (do_prefill) {
    auto last = Prefill(ex, std::vector<int>(prompt, prompt + n_prompt), bos, /*wait_for_completion=*/true, info);
    if (!last.ok()) return Finish(last.status(), err);
    res->last_prefill_id = *last;
  }
  StopTokenDetector detector(1);
  if (n_stop > 0) {
    Status s = detector.AddStopTokenSequence(std::vector<int>(stop_seq, stop_seq + n_stop));
    if (!s.ok()) return Finish(s, err);
  }
  std::vector<int> tokens;
  if (streaming) {
    Status s = DecodeStreaming(
        ex, detector, info, [&](int id) { tokens.push_back(id); },
        [&](const Status& e) { res->cache_full_error |= e.message() == "Maximum kv-cache size reached." ? 1 : 0; });
    if (!s.ok()) return Finish(s, err);
  } else {
    auto r = Decode(ex, detector, info);
    if (!r.ok()) return Finish(r.status(), err);
    tokens = *r;
  }
  res->n_tokens = static_cast<int>(tokens.size());
  for (int i = 0; i < res->n_tokens && i < cap; ++i) out_tokens[i] = tokens[i];
  res->current_step = *ex.GetCurrentStep();
  if (report && info.has_value()) {
    std::ostringstream os;
    os << *info;
    *report = CopyText(os.str());
  }
  return 0;
}
}  // namespace

// The loop over a scripted executor: expected_prefill (n_expected ids) is what Prefill must receive,
// decode_script the ids Decode hands out; max_num_tokens 0 keeps the fake's 1024.
int hle_fake_loop(const int32_t* prompt, int32_t n_prompt, int32_t bos, const int32_t* expected_prefill,
                  int32_t n_expected, const int32_t* decode_script, int32_t n_decode, int32_t max_num_tokens,
                  const int32_t* stop_seq, int32_t n_stop, int32_t bench_prefill, int32_t bench_decode,
                  int32_t streaming, int32_t do_prefill, int32_t* out_tokens, int32_t cap, hle_loop_result* res,
                  char** report, char** err) {
  std::vector<std::vector<int>> decode_set;
  for (int i = 0; i < n_decode; ++i) decode_set.push_back({decode_script[i]});
  FakeLlmExecutor ex(/*vocab_size=*/2560, {std::vector<int>(expected_prefill, expected_prefill + n_expected)}, decode_set);
  if (max_num_tokens > 0) ex.GetMutableExecutorSettings()->SetMaxNumTokens(max_num_tokens);
  return RunLoop(ex, prompt, n_prompt, bos, stop_seq, n_stop, bench_prefill, bench_decode, streaming, do_prefill,
                 out_tokens, cap, res, report, err);
}

// The reference's benchmark protocol on a HipLlmExecutor: one prefill turn of bench_prefill ids, then
// bench_decode decode steps; *report receives the BenchmarkInfo text (malloc'd).
int hle_run_benchmark(void* h, const int32_t* prompt, int32_t n_prompt, int32_t bench_prefill, int32_t bench_decode,
                      int32_t* out_tokens, int32_t cap, hle_loop_result* res, char** report, char** err) {
  const int32_t never = -1;  // a stop sequence no id matches: the step counts of the benchmark end the loop
  return RunLoop(*static_cast<HipLlmExecutor*>(h), prompt, n_prompt, /*bos=*/2, &never, 1, bench_prefill, bench_decode,
                 /*streaming=*/0, /*do_prefill=*/1, out_tokens, cap, res, report, err);
}

}  // extern "C"

// ---- .litertlm container reader (test surface)

namespace {
std::string JsonString(const std::string& text) {
  std::string out = "\"";
  for (unsigned char c : text) {
    if (c == '"' || c == '\\') {
      out.push_back('\\');
      out.push_back(static_cast<char>(c));
    } else if (c < 0x20) {
      char buf[8];
      snprintf(buf, sizeof(buf), "\\u%04x", c);
      out += buf;
    } else {
      out.push_back(static_cast<char>(c));
    }
  }
  return out + "\"";
}
std::string JsonItems(const std::vector<schema::KeyValue>& items) {
  std::string out = "[";
  for (size_t i = 0; i < items.size(); ++i) {
    const schema::KeyValue& kv = items[i];
    out += std::string(i ? ", " : "") + "{\"key\": " + JsonString(kv.key) + ", \"type\": " + std::to_string(kv.type) +
           ", \"value\": " + JsonString(kv.ToString()) + "}";
  }
  return out + "]";
}
std::string DescribeHeader(const schema::LitertlmHeader& h) {
  std::string out = "{\"version\": [" + std::to_string(h.major_version) + ", " + std::to_string(h.minor_version) + ", " +
                    std::to_string(h.patch_version) + "], \"header_end_offset\": " + std::to_string(h.header_end_offset) +
                    ", \"system_metadata\": " + JsonItems(h.system_metadata) + ", \"sections\": [";
  for (size_t i = 0; i < h.sections.size(); ++i) {
    const schema::SectionObject& s = h.sections[i];
    out += std::string(i ? ", " : "") + "{\"begin_offset\": " + std::to_string(s.begin_offset) +
           ", \"end_offset\": " + std::to_string(s.end_offset) + ", \"data_type\": " + std::to_string(s.data_type) +
           ", \"data_type_name\": " + JsonString(schema::AnySectionDataTypeToString(s.data_type)) +
           ", \"items\": " + JsonItems(s.items) + "}";
  }
  return out + "]}";
}
int GiveBytes(const Status& s, std::string& bytes, uint8_t** data, uint64_t* length, char** err) {
  if (s.ok()) {
    *length = bytes.size();
    *data = static_cast<uint8_t*>(malloc(bytes.size() ? bytes.size() : 1));
    if (*data) memcpy(*data, bytes.data(), bytes.size());
  }
  return Finish(s, err);
}
}  // namespace

extern "C" {

// The header of a .litertlm file (path != null) or of a buffer, as JSON text (malloc'd).
// The section map and token capacity an executor takes from a model file: *json receives
// {"sections": {"<kind>": [begin, end], ...}, "metadata_max_num_tokens": n, "max_num_tokens": what the settings end up with
// when they arrive holding `preset_max_num_tokens` (0 = not set)}.
int hle_model_file(const char* path, int32_t preset_max_num_tokens, char** json, char** err) {
  auto file = LitertLmModelFile::Open(path);
  if (!file.ok()) return Finish(file.status(), err);
  auto from_metadata = file->MetadataMaxNumTokens();
  if (!from_metadata.ok()) return Finish(from_metadata.status(), err);
  auto settings = LlmExecutorSettings::CreateDefault(Backend::GPU_HIP);
  if (!settings.ok()) return Finish(settings.status(), err);
  settings->SetMaxNumTokens(preset_max_num_tokens);
  Status s = file->UpdateExecutorSettings(&*settings);
  if (!s.ok()) return Finish(s, err);
  std::ostringstream os;
  os << "{\"sections\": {";
  bool first = true;
  auto put = [&](const std::string& name, const std::optional<SectionRange>& r) {
    if (!r.has_value()) return;
    os << (first ? "" : ", ") << "\"" << name << "\": [" << r->begin << ", " << r->end << "]";
    first = false;
  };
  for (ModelType t : {ModelType::kTfLitePrefillDecode, ModelType::kTfLiteEmbedder, ModelType::kTfLitePerLayerEmbedder,
                      ModelType::kTfLiteAux})
    put(ModelTypeToString(t), file->GetTFLiteModel(t));
  put("SP_Tokenizer", file->GetSentencePieceTokenizer());
  put("HF_Tokenizer_Zlib", file->GetHuggingFaceTokenizer());
  put("LlmMetadataProto", file->GetLlmMetadata());
  os << "}, \"metadata_max_num_tokens\": " << *from_metadata << ", \"max_num_tokens\": " << settings->GetMaxNumTokens() << "}";
  *json = CopyText(os.str());
  return 0;
}
// int32 varint field of a serialized protocol buffer; *value receives it (0 if absent).
int hle_proto_int32_field(const void* data, uint64_t length, int32_t field_number, int32_t* value, char** err) {
  auto r = ReadProtoInt32Field(std::string(static_cast<const char*>(data), static_cast<size_t>(length)), field_number);
  if (!r.ok()) return Finish(r.status(), err);
  *value = *r;
  return 0;
}

int hle_litertlm_header(const char* path, const void* data, uint64_t length, char** json, char** err) {
  schema::LitertlmHeader header;
  Status s = path ? schema::ReadHeaderFromLiteRTLM(std::string(path), &header)
                  : schema::ReadHeaderFromLiteRTLM(data, static_cast<size_t>(length), &header);
  if (s.ok()) *json = CopyText(DescribeHeader(header));
  return Finish(s, err);
}

// what: 0 section bytes of `expected_type`, 1 HF tokenizer JSON of section idx, 2 the first HF tokenizer JSON,
// 3 the first generic binary section. *data is malloc'd.
int hle_litertlm_read(const char* path, int32_t what, int32_t section_idx, int32_t expected_type, uint8_t** data,
                      uint64_t* length, char** err) {
  std::string bytes;
  Status s;
  switch (what) {
    case 0: s = schema::ReadSectionBytes(path, section_idx, static_cast<uint8_t>(expected_type), &bytes); break;
    case 1: s = schema::ReadHfTokenizerJsonFromSection(path, section_idx, &bytes); break;
    case 2: s = schema::ReadAnyHfTokenizerJson(path, &bytes); break;
    case 3: s = schema::ReadAnyBinaryData(path, &bytes); break;
    default: s = InvalidArgumentError("unknown read");
  }
  return GiveBytes(s, bytes, data, length, err);
}

}  // extern "C"
