// Driver around the reference's own GGUF reader -- TEST INFRASTRUCTURE ONLY.
//
// Compiled together with the reference source where it lies
// (interface/loader/gguf/gguf_reader.cpp) into oracle/_ref/libcut_ref.so by
// oracle/Makefile.  The reference's dequantizers are private statics that are
// reachable only through read_tensor_f32 on a file, so each call writes a
// one-tensor GGUF v3 file (layout parsed by gguf_reader.cpp:15-58, 281-311),
// opens it with the reference reader and returns what the reader produced.
// Nothing of the reference is copied here; this file only calls its public API.
#include "gguf_reader.hpp"

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <unistd.h>
#include <vector>

namespace {

std::string write_one_tensor_file(uint32_t ggml_type, const uint8_t *data,
                                  size_t nbytes, uint64_t rows, uint64_t cols) {
  char path[] = "/tmp/cut_ref_XXXXXX";
  int fd = mkstemp(path);
  if (fd < 0)
    return "";
  FILE *f = fdopen(fd, "wb");
  auto w32 = [&](uint32_t v) { fwrite(&v, 4, 1, f); };
  auto w64 = [&](uint64_t v) { fwrite(&v, 8, 1, f); };
  w32(gguf::GGUF_MAGIC);
  w32(3);
  w64(1); // tensor count
  w64(0); // metadata kv count
  const char name[] = "t";
  w64(1);
  fwrite(name, 1, 1, f);
  w32(2);
  w64(cols); // innermost first
  w64(rows);
  w32(ggml_type);
  w64(0); // offset in the data section
  long pos = ftell(f);
  long aligned = (pos + 31) / 32 * 32;
  for (long i = pos; i < aligned; ++i)
    fputc(0, f);
  fwrite(data, 1, nbytes, f);
  fclose(f);
  return path;
}

} // namespace

extern "C" {

// ggml_type: 2 Q4_0, 8 Q8_0, 12 Q4_K, 14 Q6_K (gguf_types.hpp:16-53).
// Returns 0 on success.
int ref_dequant(uint32_t ggml_type, const uint8_t *data, size_t nbytes,
                uint64_t rows, uint64_t cols, float *out) {
  std::string path = write_one_tensor_file(ggml_type, data, nbytes, rows, cols);
  if (path.empty())
    return -1;
  int rc = 0;
  try {
    gguf::GGUFReader reader(path);
    std::vector<float> v = reader.read_tensor_f32("t");
    if (v.size() != rows * cols)
      rc = -2;
    else
      std::memcpy(out, v.data(), v.size() * sizeof(float));
  } catch (const std::exception &e) {
    std::fprintf(stderr, "ref_dequant: %s\n", e.what());
    rc = -3;
  }
  unlink(path.c_str());
  return rc;
}

int ref_split_q8(const uint8_t *data, size_t nbytes, uint64_t rows,
                 uint64_t cols, int8_t *values, uint16_t *scales) {
  std::string path = write_one_tensor_file(8, data, nbytes, rows, cols);
  if (path.empty())
    return -1;
  int rc = 0;
  try {
    gguf::GGUFReader reader(path);
    auto s = reader.read_tensor_q8_separated("t");
    std::memcpy(values, s.values.data(), s.values.size());
    std::memcpy(scales, s.scales.data(), s.scales.size() * 2);
  } catch (const std::exception &e) {
    std::fprintf(stderr, "ref_split_q8: %s\n", e.what());
    rc = -3;
  }
  unlink(path.c_str());
  return rc;
}

int ref_split_q4(const uint8_t *data, size_t nbytes, uint64_t rows,
                 uint64_t cols, uint8_t *packed, uint16_t *scales) {
  std::string path = write_one_tensor_file(2, data, nbytes, rows, cols);
  if (path.empty())
    return -1;
  int rc = 0;
  try {
    gguf::GGUFReader reader(path);
    auto s = reader.read_tensor_q4_separated("t");
    std::memcpy(packed, s.packedValues.data(), s.packedValues.size());
    std::memcpy(scales, s.scales.data(), s.scales.size() * 2);
  } catch (const std::exception &e) {
    std::fprintf(stderr, "ref_split_q4: %s\n", e.what());
    rc = -3;
  }
  unlink(path.c_str());
  return rc;
}

// Opens `path` with the reference reader and copies the raw bytes of tensor
// `name` to out (cap bytes).  Returns the tensor's byte size, or -1.
// dims_out (if not null) receives up to 4 dimensions, innermost first; type_out the GGML type.
long ref_read_raw(const char *path, const char *name, uint8_t *out, size_t cap,
                  uint64_t *dims_out, uint32_t *type_out) {
  try {
    gguf::GGUFReader reader(path);
    std::vector<uint8_t> raw = reader.read_tensor_raw(name);
    if (raw.size() > cap)
      return -1;
    memcpy(out, raw.data(), raw.size());
    const auto &info = reader.tensors().at(name);
    if (dims_out)
      for (size_t i = 0; i < info.dimensions.size() && i < 4; ++i)
        dims_out[i] = info.dimensions[i];
    if (type_out)
      *type_out = static_cast<uint32_t>(info.type);
    return (long)raw.size();
  } catch (...) {
    return -1;
  }
}

// A uint32 metadata value read by the reference reader (0xFFFFFFFF if absent or of another type).
uint32_t ref_meta_u32(const char *path, const char *key) {
  try {
    gguf::GGUFReader reader(path);
    return reader.metadata().get_as<uint32_t>(key, 0xFFFFFFFFu);
  } catch (...) {
    return 0xFFFFFFFFu;
  }
}
}
