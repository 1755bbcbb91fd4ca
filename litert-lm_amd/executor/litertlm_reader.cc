#include "litertlm_reader.h"

#include <zlib.h>

#include <cstring>
#include <fstream>
#include <memory>

namespace litert::lm::schema {
namespace {

// Bounds-checked view of a FlatBuffer. Tables are addressed by the position of
// their first byte (where the signed offset to the vtable sits).
class Wire {
 public:
  Wire(const uint8_t* p, size_t n) : p_(p), n_(n) {}
  bool ok() const { return ok_; }

  template <class T>
  T Read(uint64_t pos) {
    T v{};
    if (pos > n_ || sizeof(T) > n_ - pos) {
      ok_ = false;
      return v;
    }
    std::memcpy(&v, p_ + pos, sizeof(T));
    return v;
  }
  // Position a forward offset stored at `pos` points to.
  uint64_t Follow(uint64_t pos) { return pos + Read<uint32_t>(pos); }
  // Position of field `index` inside the table at `table`, 0 if the field is absent.
  uint64_t Field(uint64_t table, int index) {
    const int64_t vtable = static_cast<int64_t>(table) - Read<int32_t>(table);
    if (vtable < 0) {
      ok_ = false;
      return 0;
    }
    const uint16_t vtable_size = Read<uint16_t>(static_cast<uint64_t>(vtable));
    const uint64_t slot = 4 + 2 * static_cast<uint64_t>(index);
    if (slot + 2 > vtable_size) return 0;
    const uint16_t off = Read<uint16_t>(static_cast<uint64_t>(vtable) + slot);
    return off ? table + off : 0;
  }
  std::string String(uint64_t field_pos) {
    const uint64_t s = Follow(field_pos);
    const uint32_t len = Read<uint32_t>(s);
    if (!ok_ || s + 4 > n_ || len > n_ - (s + 4)) {
      ok_ = false;
      return std::string();
    }
    return std::string(reinterpret_cast<const char*>(p_ + s + 4), len);
  }
  // Positions of the elements of a vector of offsets (tables / strings).
  std::vector<uint64_t> TableVector(uint64_t field_pos) {
    std::vector<uint64_t> out;
    const uint64_t v = Follow(field_pos);
    const uint32_t count = Read<uint32_t>(v);
    if (!ok_ || v + 4 > n_ || static_cast<uint64_t>(count) * 4 > n_ - (v + 4)) {
      ok_ = false;
      return out;
    }
    for (uint32_t i = 0; i < count; ++i) out.push_back(Follow(v + 4 + 4 * static_cast<uint64_t>(i)));
    return out;
  }

 private:
  const uint8_t* p_;
  size_t n_;
  bool ok_ = true;
};

// KeyValuePair { key: string; value_type: ubyte; value: union } (fields 0, 1, 2).
KeyValue ReadKeyValue(Wire& w, uint64_t table) {
  KeyValue kv;
  if (const uint64_t key = w.Field(table, 0)) kv.key = w.String(key);
  if (const uint64_t type = w.Field(table, 1)) kv.type = w.Read<uint8_t>(type);
  const uint64_t value_field = w.Field(table, 2);
  if (!value_field || kv.type == VData_NONE) return kv;
  const uint64_t value = w.Follow(value_field);  // a struct (scalars in place) or the StringValue table
  switch (kv.type) {
    case VData_UInt8: kv.u = w.Read<uint8_t>(value); break;
    case VData_Int8: kv.i = w.Read<int8_t>(value); break;
    case VData_UInt16: kv.u = w.Read<uint16_t>(value); break;
    case VData_Int16: kv.i = w.Read<int16_t>(value); break;
    case VData_UInt32: kv.u = w.Read<uint32_t>(value); break;
    case VData_Int32: kv.i = w.Read<int32_t>(value); break;
    case VData_Float32: kv.f = w.Read<float>(value); break;
    case VData_Bool: kv.i = w.Read<uint8_t>(value) != 0; break;
    case VData_StringValue:
      if (const uint64_t s = w.Field(value, 0)) kv.s = w.String(s);
      break;
    case VData_UInt64: kv.u = w.Read<uint64_t>(value); break;
    case VData_Int64: kv.i = w.Read<int64_t>(value); break;
    default: break;  // a type newer than this reader: key and type are kept
  }
  return kv;
}

Status ReadFileRange(const std::string& path, uint64_t begin, uint64_t end, std::string* out) {
  std::ifstream in(path, std::ios::binary);
  if (!in.is_open()) return InternalError("Could not open file: " + path);
  // offsets come from the file's own header: they are checked against the file before anything is sized by them
  in.seekg(0, std::ios::end);
  const std::streamoff file_size = in.tellg();
  if (file_size < 0) return InternalError("Could not size file: " + path);
  if (end < begin)
    return InvalidArgumentError("Section range [" + std::to_string(begin) + ", " + std::to_string(end) + ") is reversed.");
  // (a file that ends before the section does: the status of a short read, without sizing anything by the header)
  if (end > static_cast<uint64_t>(file_size))
    return InternalError("Could not read " + std::to_string(end - begin) + " bytes from stream.");
  in.seekg(static_cast<std::streamoff>(begin));
  out->resize(end - begin);
  in.read(out->data(), static_cast<std::streamsize>(out->size()));
  if (!in) return InternalError("Could not read " + std::to_string(out->size()) + " bytes from stream.");
  return OkStatus();
}

}  // namespace

std::string AnySectionDataTypeToString(uint8_t type) {
  static const char* const kNames[] = {"NONE",         "GenericBinaryData", "Deprecated",       "TFLiteModel",
                                       "SP_Tokenizer", "LlmMetadataProto",  "HF_Tokenizer_Zlib"};
  return type < 7 ? kNames[type] : "Unknown(" + std::to_string(type) + ")";
}

std::string KeyValue::ToString() const {
  switch (type) {
    case VData_UInt8: case VData_UInt16: case VData_UInt32: case VData_UInt64: return std::to_string(u);
    case VData_Int8: case VData_Int16: case VData_Int32: case VData_Int64: return std::to_string(i);
    case VData_Float32: return std::to_string(f);
    case VData_Bool: return i ? "true" : "false";
    case VData_StringValue: return s;
    default: return "";
  }
}

Status ReadHeaderFromLiteRTLM(const void* data, size_t length, LitertlmHeader* header) {
  const uint8_t* p = static_cast<const uint8_t*>(data);
  if (length < 8 || std::memcmp(p, "LITERTLM", 8) != 0)
    return InvalidArgumentError("Invalid magic number or failed to read: " +
                                std::string(reinterpret_cast<const char*>(p), length < 8 ? length : 8));
  if (length < 20) return InternalError("Failed to read version bytes.");
  std::memcpy(&header->major_version, p + 8, 4);
  std::memcpy(&header->minor_version, p + 12, 4);
  std::memcpy(&header->patch_version, p + 16, 4);
  if (header->major_version != LITERTLM_MAJOR_VERSION)
    return UnimplementedError("Unimplemented Error: This reader doesn't support version " +
                              std::to_string(header->major_version) + ", expected version " +
                              std::to_string(LITERTLM_MAJOR_VERSION) + ".");
  if (length < 24) return InternalError("Failed to skip padding after version.");
  if (length < 32) return InternalError("Failed to read header end offset.");
  std::memcpy(&header->header_end_offset, p + 24, 8);
  if (header->header_end_offset < 32)
    return InvalidArgumentError("Invalid header end offset: smaller than current position.");
  if (header->header_end_offset > length) return InternalError("Failed to read header data.");

  Wire w(p + 32, static_cast<size_t>(header->header_end_offset - 32));
  header->system_metadata.clear();
  header->sections.clear();
  const uint64_t root = w.Follow(0);  // LiteRTLMMetaData { system_metadata, section_metadata }
  if (const uint64_t sys_field = w.Field(root, 0)) {
    const uint64_t sys = w.Follow(sys_field);  // SystemMetadata { entries }
    if (const uint64_t entries = w.Field(sys, 0))
      for (uint64_t kv : w.TableVector(entries)) header->system_metadata.push_back(ReadKeyValue(w, kv));
  }
  if (const uint64_t sec_field = w.Field(root, 1)) {
    const uint64_t sec = w.Follow(sec_field);  // SectionMetadata { objects }
    if (const uint64_t objects = w.Field(sec, 0)) {
      for (uint64_t obj : w.TableVector(objects)) {  // SectionObject { items, begin_offset, end_offset, data_type }
        SectionObject s;
        if (const uint64_t items = w.Field(obj, 0))
          for (uint64_t kv : w.TableVector(items)) s.items.push_back(ReadKeyValue(w, kv));
        if (const uint64_t f = w.Field(obj, 1)) s.begin_offset = w.Read<uint64_t>(f);
        if (const uint64_t f = w.Field(obj, 2)) s.end_offset = w.Read<uint64_t>(f);
        if (const uint64_t f = w.Field(obj, 3)) s.data_type = w.Read<uint8_t>(f);
        header->sections.push_back(std::move(s));
      }
    }
  }
  if (!w.ok()) return InvalidArgumentError("Malformed header: an offset points outside the header.");
  return OkStatus();
}

Status ReadHeaderFromLiteRTLM(const std::string& litertlm_path, LitertlmHeader* header) {
  std::ifstream in(litertlm_path, std::ios::binary);
  if (!in.is_open()) return InternalError("Could not open file: " + litertlm_path);
  // preamble first, then exactly the header bytes it announces
  std::string buf(32, '\0');
  in.read(buf.data(), 32);
  const size_t got = static_cast<size_t>(in.gcount());
  if (got < 32) return ReadHeaderFromLiteRTLM(buf.data(), got, header);
  uint64_t header_end = 0;
  std::memcpy(&header_end, buf.data() + 24, 8);
  if (header_end > 32 && header_end <= (64u << 20) && std::memcmp(buf.data(), "LITERTLM", 8) == 0) {
    buf.resize(static_cast<size_t>(header_end));
    in.read(buf.data() + 32, static_cast<std::streamsize>(header_end - 32));
    buf.resize(32 + static_cast<size_t>(in.gcount()));
  }
  return ReadHeaderFromLiteRTLM(buf.data(), buf.size(), header);
}

Status ReadSectionBytes(const std::string& litertlm_path, int section_idx, uint8_t expected_type, std::string* data) {
  LitertlmHeader header;
  RETURN_IF_ERROR(ReadHeaderFromLiteRTLM(litertlm_path, &header));
  const int count = static_cast<int>(header.sections.size());
  if (section_idx < 0 || section_idx >= count)
    return InvalidArgumentError("Invalid section index: " + std::to_string(section_idx) +
                                ", num sections = " + std::to_string(count));
  const SectionObject& s = header.sections[section_idx];
  if (s.data_type != expected_type)
    return InvalidArgumentError("Section " + std::to_string(section_idx) + " is not the expected type.  It is: " +
                                AnySectionDataTypeToString(s.data_type) + ", expected " + std::to_string(expected_type));
  if (s.end_offset < s.begin_offset)
    return InvalidArgumentError("Section " + std::to_string(section_idx) + " ends before it begins.");
  if (s.end_offset == s.begin_offset)
    return InvalidArgumentError("Section " + std::to_string(section_idx) + " has zero size.");
  return ReadFileRange(litertlm_path, s.begin_offset, s.end_offset, data);
}

Status ReadBinaryDataFromSection(const std::string& litertlm_path, int section_idx, std::string* data) {
  return ReadSectionBytes(litertlm_path, section_idx, AnySectionDataType_GenericBinaryData, data);
}

Status ReadHfTokenizerJsonFromSection(const std::string& litertlm_path, int section_idx, std::string* json) {
  std::string packed;
  RETURN_IF_ERROR(ReadSectionBytes(litertlm_path, section_idx, AnySectionDataType_HF_Tokenizer_Zlib, &packed));
  if (packed.size() < sizeof(uint64_t)) return InternalError("Data too short to contain compressed size.");
  uint64_t size = 0;
  std::memcpy(&size, packed.data(), sizeof(uint64_t));
  if (size > (1ull << 32)) return InternalError("Implausible uncompressed size " + std::to_string(size) + ".");
  std::string out(static_cast<size_t>(size), '\0');
  uLongf out_len = static_cast<uLongf>(size);
  const int rc = uncompress(reinterpret_cast<Bytef*>(out.data()), &out_len,
                            reinterpret_cast<const Bytef*>(packed.data() + sizeof(uint64_t)),
                            static_cast<uLong>(packed.size() - sizeof(uint64_t)));
  switch (rc) {
    case Z_OK:
      out.resize(out_len);
      *json = std::move(out);
      return OkStatus();
    case Z_BUF_ERROR: return InternalError("Output buffer was not large enough.");
    case Z_MEM_ERROR: return InternalError("Not enough memory to decompress.");
    case Z_DATA_ERROR: return InternalError("Invalid or incomplete compressed data.");
    default: return InternalError("Unknown decompression error " + std::to_string(rc));
  }
}

StatusOr<int> FindFirstSection(const LitertlmHeader& header, uint8_t type) {
  for (size_t i = 0; i < header.sections.size(); ++i)
    if (header.sections[i].data_type == type) return static_cast<int>(i);
  return NotFoundError("No matching section found in the file.");
}

Status ReadAnyHfTokenizerJson(const std::string& litertlm_path, std::string* json) {
  LitertlmHeader header;
  RETURN_IF_ERROR(ReadHeaderFromLiteRTLM(litertlm_path, &header));
  ASSIGN_OR_RETURN(const int idx, FindFirstSection(header, AnySectionDataType_HF_Tokenizer_Zlib));
  return ReadHfTokenizerJsonFromSection(litertlm_path, idx, json);
}

Status ReadAnyBinaryData(const std::string& litertlm_path, std::string* data) {
  LitertlmHeader header;
  RETURN_IF_ERROR(ReadHeaderFromLiteRTLM(litertlm_path, &header));
  ASSIGN_OR_RETURN(const int idx, FindFirstSection(header, AnySectionDataType_GenericBinaryData));
  return ReadBinaryDataFromSection(litertlm_path, idx, data);
}

}  // namespace litert::lm::schema
