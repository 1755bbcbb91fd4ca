#include "model_file.h"

#include <algorithm>
#include <cctype>
#include <fstream>

namespace litert::lm {
namespace {

std::string Lower(std::string text) {
  std::transform(text.begin(), text.end(), text.begin(), [](unsigned char c) { return static_cast<char>(std::tolower(c)); });
  return text;
}

// One base-128 varint at `*at`; false when the message ends inside it or it runs past ten bytes.
bool ReadVarint(const std::string& m, size_t* at, uint64_t* value) {
  uint64_t v = 0;
  for (int shift = 0; shift < 70; shift += 7) {
    if (*at >= m.size()) return false;
    const uint8_t byte = static_cast<uint8_t>(m[(*at)++]);
    v |= static_cast<uint64_t>(byte & 0x7F) << (shift < 64 ? shift : 63);
    if (!(byte & 0x80)) {
      *value = v;
      return true;
    }
  }
  return false;
}

}  // namespace

StatusOr<ModelType> StringToModelType(const std::string& text) {
  const std::string lower = Lower(text);
  if (lower == "tf_lite_prefill_decode") return ModelType::kTfLitePrefillDecode;
  if (lower == "tf_lite_embedder") return ModelType::kTfLiteEmbedder;
  if (lower == "tf_lite_per_layer_embedder") return ModelType::kTfLitePerLayerEmbedder;
  if (lower == "tf_lite_aux") return ModelType::kTfLiteAux;
  return InvalidArgumentError("Unknown model type: " + text);
}

std::string ModelTypeToString(ModelType type) {
  switch (type) {
    case ModelType::kTfLitePrefillDecode: return "TF_LITE_PREFILL_DECODE";
    case ModelType::kTfLiteEmbedder: return "TF_LITE_EMBEDDER";
    case ModelType::kTfLitePerLayerEmbedder: return "TF_LITE_PER_LAYER_EMBEDDER";
    case ModelType::kTfLiteAux: return "TF_LITE_AUX";
    case ModelType::kUnknown: return "UNKNOWN";
  }
  return "INVALID";
}

StatusOr<int32_t> ReadProtoInt32Field(const std::string& message, int field_number) {
  int32_t found = 0;
  size_t at = 0;
  while (at < message.size()) {
    uint64_t tag = 0;
    if (!ReadVarint(message, &at, &tag)) return InvalidArgumentError("protocol buffer: truncated field tag.");
    const uint64_t field = tag >> 3;
    const int wire = static_cast<int>(tag & 7);
    if (field == 0) return InvalidArgumentError("protocol buffer: field number 0.");
    uint64_t value = 0;
    switch (wire) {
      case 0:  // varint
        if (!ReadVarint(message, &at, &value)) return InvalidArgumentError("protocol buffer: truncated varint.");
        if (field == static_cast<uint64_t>(field_number)) found = static_cast<int32_t>(value);  // (int32: the low 32 bits)
        break;
      case 1:  // 64 bits
        if (message.size() - at < 8) return InvalidArgumentError("protocol buffer: truncated 64-bit field.");
        at += 8;
        break;
      case 2:  // length-delimited
        if (!ReadVarint(message, &at, &value) || message.size() - at < value)
          return InvalidArgumentError("protocol buffer: length-delimited field runs past the message.");
        at += static_cast<size_t>(value);
        break;
      case 5:  // 32 bits
        if (message.size() - at < 4) return InvalidArgumentError("protocol buffer: truncated 32-bit field.");
        at += 4;
        break;
      default:
        return InvalidArgumentError("protocol buffer: wire type " + std::to_string(wire) + " is not supported.");
    }
  }
  return found;
}

StatusOr<LitertLmModelFile> LitertLmModelFile::Open(const std::string& path) {
  LitertLmModelFile file;
  file.path_ = path;
  RETURN_IF_ERROR(schema::ReadHeaderFromLiteRTLM(path, &file.header_));
  std::ifstream in(path, std::ios::binary | std::ios::ate);
  if (!in) return NotFoundError("Could not open " + path);
  const uint64_t file_size = static_cast<uint64_t>(in.tellg());
  for (size_t i = 0; i < file.header_.sections.size(); ++i) {
    const schema::SectionObject& section = file.header_.sections[i];
    if (section.begin_offset > section.end_offset || section.end_offset > file_size)
      return InvalidArgumentError("Section " + std::to_string(i) + " [" + std::to_string(section.begin_offset) + ", " +
                                  std::to_string(section.end_offset) + ") does not lie inside the file (" +
                                  std::to_string(file_size) + " bytes).");
    ModelType type = ModelType::kUnknown;
    if (section.data_type == schema::AnySectionDataType_TFLiteModel) {
      type = ModelType::kTfLitePrefillDecode;  // sections written before the item existed
      for (const schema::KeyValue& item : section.items) {
        if (Lower(item.key) != "model_type" || item.type != schema::VData_StringValue) continue;
        ASSIGN_OR_RETURN(type, StringToModelType(item.s));
        break;
      }
    }
    file.sections_[Key(section.data_type, type)] = SectionRange{section.begin_offset, section.end_offset};
  }
  return file;
}

std::optional<SectionRange> LitertLmModelFile::Find(uint8_t data_type, ModelType type) const {
  const auto it = sections_.find(Key(data_type, type));
  if (it == sections_.end()) return std::nullopt;
  return it->second;
}

std::optional<SectionRange> LitertLmModelFile::GetTFLiteModel(ModelType type) const {
  return Find(schema::AnySectionDataType_TFLiteModel, type);
}

StatusOr<int> LitertLmModelFile::MetadataMaxNumTokens() const {
  const std::optional<SectionRange> range = GetLlmMetadata();
  if (!range.has_value()) return 0;
  std::ifstream in(path_, std::ios::binary);
  if (!in) return NotFoundError("Could not open " + path_);
  std::string message(static_cast<size_t>(range->size()), '\0');
  in.seekg(static_cast<std::streamoff>(range->begin));
  in.read(message.data(), static_cast<std::streamsize>(message.size()));
  if (static_cast<uint64_t>(in.gcount()) != range->size()) return InternalError("Could not read the LlmMetadata section.");
  ASSIGN_OR_RETURN(const int32_t value, ReadProtoInt32Field(message, /*max_num_tokens=*/5));
  return static_cast<int>(value);
}

Status LitertLmModelFile::UpdateExecutorSettings(LlmExecutorSettings* settings) const {
  if (settings->GetMaxNumTokens() != 0) return OkStatus();
  ASSIGN_OR_RETURN(const int from_file, MetadataMaxNumTokens());
  settings->SetMaxNumTokens(from_file > 0 ? from_file : 4096);
  return OkStatus();
}

}  // namespace litert::lm
