// What an executor takes from a .litertlm model file before it runs: where the sections are and how many tokens
// the model holds. The section map follows LitertLmLoader::MapSections (runtime/util/litert_lm_loader.cc:57-115:
// a section is filed under its data type, a TFLite model section under its data type and the model type its
// "model_type" item names, tf_lite_prefill_decode when it names none; a later section of the same kind replaces
// an earlier one), the accessors LitertLmLoader's getters (litert_lm_loader.h), and the token capacity
// EngineSettings::MaybeUpdateAndValidate (runtime/engine/engine_settings.cc:79-88: the settings' own value if set,
// else LlmMetadata.max_num_tokens if positive, else 4096). LlmMetadata is a protocol buffer
// (runtime/proto/llm_metadata.proto:46-62); only its int32 field 5 is read, straight from the wire format.
#ifndef LITERT_LM_AMD_EXECUTOR_MODEL_FILE_H_
#define LITERT_LM_AMD_EXECUTOR_MODEL_FILE_H_

#include <cstdint>
#include <map>
#include <optional>
#include <string>
#include <utility>

#include "litertlm_reader.h"
#include "llm_executor_settings.h"
#include "status.h"

namespace litert::lm {

// runtime/components/model_resources.h:34-77.
enum class ModelType { kUnknown = 0, kTfLitePrefillDecode = 1, kTfLiteEmbedder = 2, kTfLitePerLayerEmbedder = 3, kTfLiteAux = 4 };
StatusOr<ModelType> StringToModelType(const std::string& text);  // case-insensitive; kInvalidArgument "Unknown model type: ..."
std::string ModelTypeToString(ModelType type);

struct SectionRange {
  uint64_t begin = 0, end = 0;  // byte offsets in the file
  uint64_t size() const { return end - begin; }
};

class LitertLmModelFile {
 public:
  // Reads the header and files the sections. Errors of the header reader pass through; a TFLite section whose
  // model type is not one of the four is kInvalidArgument; offsets beyond the file are kInvalidArgument.
  static StatusOr<LitertLmModelFile> Open(const std::string& path);

  const std::string& path() const { return path_; }
  const schema::LitertlmHeader& header() const { return header_; }
  std::optional<SectionRange> GetTFLiteModel(ModelType type) const;
  std::optional<SectionRange> GetSentencePieceTokenizer() const { return Find(schema::AnySectionDataType_SP_Tokenizer); }
  std::optional<SectionRange> GetHuggingFaceTokenizer() const { return Find(schema::AnySectionDataType_HF_Tokenizer_Zlib); }
  std::optional<SectionRange> GetLlmMetadata() const { return Find(schema::AnySectionDataType_LlmMetadataProto); }

  // LlmMetadata.max_num_tokens of the file's metadata section; 0 when the file has no such section or the
  // message does not set the field. kInvalidArgument for a message that does not parse.
  StatusOr<int> MetadataMaxNumTokens() const;
  // The token capacity rule: leaves a value the caller has set, else the metadata's if positive, else 4096.
  Status UpdateExecutorSettings(LlmExecutorSettings* settings) const;

 private:
  using Key = std::pair<uint8_t, ModelType>;  // (AnySectionDataType, model type: kUnknown for everything but models)
  std::optional<SectionRange> Find(uint8_t data_type, ModelType type = ModelType::kUnknown) const;
  std::string path_;
  schema::LitertlmHeader header_;
  std::map<Key, SectionRange> sections_;
};

// int32 field `field_number` (wire type varint) of a serialized message: the last occurrence, 0 if absent.
StatusOr<int32_t> ReadProtoInt32Field(const std::string& message, int field_number);

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_MODEL_FILE_H_
