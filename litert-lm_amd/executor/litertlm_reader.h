// Reader of the .litertlm container: fixed preamble, FlatBuffers header with the
// system metadata and the section map, then the sections themselves at the
// offsets the map names (schema/core/litertlm_header_schema.fbs:18-104,
// schema/core/litertlm_read.cc:37-330 of the reference). The header is decoded
// here directly from the FlatBuffers wire format (no generated code, every
// offset bounds-checked), which is all that is needed to find the tokenizer,
// the metadata and the model sections of a file.
//
//   bytes 0..7    "LITERTLM"
//   bytes 8..19   major, minor, patch version (uint32 little endian)
//   bytes 20..23  padding
//   bytes 24..31  offset of the end of the header (uint64)
//   bytes 32..    LiteRTLMMetaData FlatBuffer { system_metadata, section_metadata }
#ifndef LITERT_LM_AMD_EXECUTOR_LITERTLM_READER_H_
#define LITERT_LM_AMD_EXECUTOR_LITERTLM_READER_H_

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "status.h"

namespace litert::lm::schema {

constexpr uint32_t LITERTLM_MAJOR_VERSION = 1;

// AnySectionDataType (litertlm_header_schema.fbs:74-82).
enum AnySectionDataType : uint8_t {
  AnySectionDataType_NONE = 0,
  AnySectionDataType_GenericBinaryData = 1,
  AnySectionDataType_Deprecated = 2,
  AnySectionDataType_TFLiteModel = 3,
  AnySectionDataType_SP_Tokenizer = 4,
  AnySectionDataType_LlmMetadataProto = 5,
  AnySectionDataType_HF_Tokenizer_Zlib = 6,
};
std::string AnySectionDataTypeToString(uint8_t type);

// VData union (litertlm_header_schema.fbs:34-46).
enum VData : uint8_t {
  VData_NONE = 0, VData_UInt8, VData_Int8, VData_UInt16, VData_Int16, VData_UInt32, VData_Int32, VData_Float32,
  VData_Bool, VData_StringValue, VData_UInt64, VData_Int64,
};

struct KeyValue {
  std::string key;
  uint8_t type = VData_NONE;
  int64_t i = 0;      // the signed integer types and Bool
  uint64_t u = 0;     // the unsigned integer types
  float f = 0.f;      // Float32
  std::string s;      // StringValue
  std::string ToString() const;  // the value as text
};

struct SectionObject {
  std::vector<KeyValue> items;
  uint64_t begin_offset = 0, end_offset = 0;
  uint8_t data_type = AnySectionDataType_NONE;
};

struct LitertlmHeader {
  uint32_t major_version = 0, minor_version = 0, patch_version = 0;
  uint64_t header_end_offset = 0;
  std::vector<KeyValue> system_metadata;
  std::vector<SectionObject> sections;
};

// kInvalidArgument: wrong magic, header end before the header's start, offsets
// that leave the buffer; kUnimplemented: another major version; kInternal:
// short reads (litertlm_read.cc:37-108).
Status ReadHeaderFromLiteRTLM(const void* data, size_t length, LitertlmHeader* header);
Status ReadHeaderFromLiteRTLM(const std::string& litertlm_path, LitertlmHeader* header);

// The bytes of section `section_idx`, which must have type `expected_type`
// (kInvalidArgument for a bad index, another type or an empty section;
// litertlm_read.cc:139-181, 258-277).
Status ReadSectionBytes(const std::string& litertlm_path, int section_idx, uint8_t expected_type, std::string* data);
Status ReadBinaryDataFromSection(const std::string& litertlm_path, int section_idx, std::string* data);
// A HF tokenizer section: uint64 uncompressed size, then a zlib stream (litertlm_read.cc:279-318).
Status ReadHfTokenizerJsonFromSection(const std::string& litertlm_path, int section_idx, std::string* json);
// The first section of the given type (ReadAny*, litertlm_read.cc:400-470); kNotFound if there is none.
StatusOr<int> FindFirstSection(const LitertlmHeader& header, uint8_t type);
Status ReadAnyHfTokenizerJson(const std::string& litertlm_path, std::string* json);
Status ReadAnyBinaryData(const std::string& litertlm_path, std::string* data);

}  // namespace litert::lm::schema
#endif  // LITERT_LM_AMD_EXECUTOR_LITERTLM_READER_H_
