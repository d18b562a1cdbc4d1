// On-disk form of a packed int4 weight: the packed nibbles, scales and zero points exactly as
// yscv_hip_int4_weight_create takes them, behind a fixed 64-byte header, so a weight that was quantised once is
// uploaded again without the f32 round trip of quantize_matmul_weights_int4_packed
// (crates/yscv-onnx/src/quantize/packed_int4.rs:50-128).  The reference keeps PackedInt4Weight in memory only
// (packed_int4.rs:29-39) and has no file format for it; this one is new.
//
// Layout (little endian):
//   0   8  magic "YSCVI4W\0"
//   8   4  version (1)
//   12  4  scale dtype (YSCV_HIP_F32 / YSCV_HIP_F16)
//   16  4  nibble format (YSCV_HIP_NIBBLE_SIGNED / _UNSIGNED)
//   20  4  1 if zero points follow, else 0
//   24  8  n (weight rows)
//   32  8  k
//   40  8  group size
//   48  8  FNV-1a 64 of the three payload sections (without their padding)
//   56  8  reserved, 0
//   64  ..  packed [n][k/2], then scales [n][k/group], then zero points [n][ceil((k/group)/2)]; every section starts
//           on a 64-byte boundary (zero padding in between).
// Everything here is host code; only yscv_hip_int4_weight_load touches the GPU (through the ordinary upload).
#include <cerrno>
#include <cstdio>
#include <vector>

#include "common.hpp"

namespace yscv {
namespace {

constexpr char kMagic[8] = {'Y', 'S', 'C', 'V', 'I', '4', 'W', '\0'};
constexpr uint32_t kVersion = 1;
constexpr size_t kHeaderBytes = 64, kAlign = 64;

struct Sections {
  size_t packed, scales, zps;  // payload bytes of each section
};

void put32(uint8_t *p, uint32_t v) {
  for (int i = 0; i < 4; i++) p[i] = (uint8_t)(v >> (8 * i));
}
void put64(uint8_t *p, uint64_t v) {
  for (int i = 0; i < 8; i++) p[i] = (uint8_t)(v >> (8 * i));
}
uint32_t get32(const uint8_t *p) {
  uint32_t v = 0;
  for (int i = 0; i < 4; i++) v |= (uint32_t)p[i] << (8 * i);
  return v;
}
uint64_t get64(const uint8_t *p) {
  uint64_t v = 0;
  for (int i = 0; i < 8; i++) v |= (uint64_t)p[i] << (8 * i);
  return v;
}
uint64_t fnv1a(uint64_t h, const void *data, size_t bytes) {
  const uint8_t *p = static_cast<const uint8_t *>(data);
  for (size_t i = 0; i < bytes; i++) {
    h ^= p[i];
    h *= 0x100000001B3ull;
  }
  return h;
}
constexpr uint64_t kFnvSeed = 0xCBF29CE484222325ull;

// Shape contract of yscv_hip_int4_weight_create, checked before anything is written or allocated.
int32_t check_shape(int32_t scale_dtype, int32_t nibble_format, bool has_zp, size_t n, size_t k, size_t g, Sections *s) {
  YSCV_REQUIRE(scale_dtype == YSCV_HIP_F32 || scale_dtype == YSCV_HIP_F16, "scale dtype must be f32 or f16, got %d", scale_dtype);
  YSCV_REQUIRE(nibble_format == YSCV_HIP_NIBBLE_SIGNED || nibble_format == YSCV_HIP_NIBBLE_UNSIGNED,
               "unknown nibble format %d", nibble_format);
  YSCV_REQUIRE(!has_zp || nibble_format == YSCV_HIP_NIBBLE_UNSIGNED, "zero points need the unsigned nibble format");
  YSCV_REQUIRE(n > 0 && k > 0 && g > 0, "empty weight: n=%zu k=%zu group=%zu", n, k, g);
  YSCV_REQUIRE(g % 2 == 0 && k % g == 0, "group size %zu must be even and divide k=%zu", g, k);
  YSCV_REQUIRE(n <= ((size_t)1 << 40) / k, "weight of %zu x %zu elements is beyond what a file may hold", n, k);
  const size_t groups = k / g;
  s->packed = n * (k / 2);
  s->scales = n * groups * (scale_dtype == YSCV_HIP_F32 ? 4 : 2);
  s->zps = has_zp ? n * ((groups + 1) / 2) : 0;
  return YSCV_HIP_OK;
}

struct File {
  FILE *f = nullptr;
  ~File() {
    if (f) fclose(f);
  }
};

int32_t write_section(FILE *f, const void *data, size_t bytes, const char *what) {
  if (bytes && fwrite(data, 1, bytes, f) != bytes) return set_error(YSCV_HIP_ERR_INVALID_ARG, "short write of %s: %s", what, strerror(errno));
  static const uint8_t zeros[kAlign] = {0};
  const size_t pad = round_up(bytes, kAlign) - bytes;
  if (pad && fwrite(zeros, 1, pad, f) != pad) return set_error(YSCV_HIP_ERR_INVALID_ARG, "short write of %s padding", what);
  return YSCV_HIP_OK;
}

int32_t read_section(FILE *f, void *dst, size_t bytes, const char *what, const char *path) {
  if (bytes && fread(dst, 1, bytes, f) != bytes) return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: file ends inside the %s", path, what);
  const size_t pad = round_up(bytes, kAlign) - bytes;
  if (pad && fseek(f, (long)pad, SEEK_CUR) != 0) return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: cannot skip the %s padding", path, what);
  return YSCV_HIP_OK;
}

int32_t read_header(FILE *f, const char *path, yscv_hip_int4_file_header *h, Sections *s) {
  uint8_t raw[kHeaderBytes];
  if (fread(raw, 1, kHeaderBytes, f) != kHeaderBytes) return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: shorter than the %zu-byte header", path, kHeaderBytes);
  if (memcmp(raw, kMagic, 8) != 0) return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: not a packed int4 weight file (bad magic)", path);
  const uint32_t version = get32(raw + 8);
  if (version != kVersion) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "%s: format version %u, this build reads %u", path, version, kVersion);
  h->scale_dtype = (int32_t)get32(raw + 12);
  h->nibble_format = (int32_t)get32(raw + 16);
  const uint32_t zp_flag = get32(raw + 20);
  if (zp_flag > 1) return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: zero-point flag %u", path, zp_flag);
  h->has_zero_points = (int32_t)zp_flag;
  h->n = get64(raw + 24);
  h->k = get64(raw + 32);
  h->group_size = get64(raw + 40);
  h->checksum = get64(raw + 48);
  YSCV_TRY(check_shape(h->scale_dtype, h->nibble_format, zp_flag != 0, (size_t)h->n, (size_t)h->k, (size_t)h->group_size, s));
  h->packed_bytes = s->packed;
  h->scales_bytes = s->scales;
  h->zero_points_bytes = s->zps;
  // the length the header implies must be the length of the file: nothing is allocated or read on the word of a
  // damaged header
  const uint64_t expect = kHeaderBytes + round_up(s->packed, kAlign) + round_up(s->scales, kAlign) + round_up(s->zps, kAlign);
  if (fseek(f, 0, SEEK_END) != 0) return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: cannot seek", path);
  const long end = ftell(f);
  if (end < 0 || (uint64_t)end != expect)
    return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: %ld bytes on disk, the header describes %llu", path, end, (unsigned long long)expect);
  if (fseek(f, (long)kHeaderBytes, SEEK_SET) != 0) return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: cannot seek", path);
  return YSCV_HIP_OK;
}

}  // namespace
}  // namespace yscv

using namespace yscv;

extern "C" {

int32_t yscv_hip_int4_file_write(const char *path, const uint8_t *packed, const void *scales, int32_t scale_dtype,
                                 const uint8_t *zero_points, int32_t nibble_format, size_t n, size_t k, size_t group_size) {
  YSCV_REQUIRE(path != nullptr && packed != nullptr && scales != nullptr, "null argument");
  Sections s{};
  YSCV_TRY(check_shape(scale_dtype, nibble_format, zero_points != nullptr, n, k, group_size, &s));
  uint64_t sum = fnv1a(kFnvSeed, packed, s.packed);
  sum = fnv1a(sum, scales, s.scales);
  if (zero_points) sum = fnv1a(sum, zero_points, s.zps);
  uint8_t raw[kHeaderBytes] = {0};
  memcpy(raw, kMagic, 8);
  put32(raw + 8, kVersion);
  put32(raw + 12, (uint32_t)scale_dtype);
  put32(raw + 16, (uint32_t)nibble_format);
  put32(raw + 20, zero_points ? 1u : 0u);
  put64(raw + 24, n);
  put64(raw + 32, k);
  put64(raw + 40, group_size);
  put64(raw + 48, sum);
  File out;
  out.f = fopen(path, "wb");
  if (!out.f) return set_error(YSCV_HIP_ERR_INVALID_ARG, "cannot create %s: %s", path, strerror(errno));
  if (fwrite(raw, 1, kHeaderBytes, out.f) != kHeaderBytes) return set_error(YSCV_HIP_ERR_INVALID_ARG, "short write of the header: %s", strerror(errno));
  YSCV_TRY(write_section(out.f, packed, s.packed, "packed nibbles"));
  YSCV_TRY(write_section(out.f, scales, s.scales, "scales"));
  if (zero_points) YSCV_TRY(write_section(out.f, zero_points, s.zps, "zero points"));
  FILE *f = out.f;
  out.f = nullptr;
  if (fclose(f) != 0) return set_error(YSCV_HIP_ERR_INVALID_ARG, "closing %s failed: %s", path, strerror(errno));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_int4_file_read_header(const char *path, yscv_hip_int4_file_header *header) {
  YSCV_REQUIRE(path != nullptr && header != nullptr, "null argument");
  File in;
  in.f = fopen(path, "rb");
  if (!in.f) return set_error(YSCV_HIP_ERR_INVALID_ARG, "cannot open %s: %s", path, strerror(errno));
  Sections s{};
  return read_header(in.f, path, header, &s);
}

int32_t yscv_hip_int4_file_read(const char *path, uint8_t *packed, size_t packed_bytes, void *scales, size_t scales_bytes,
                                uint8_t *zero_points, size_t zero_points_bytes) {
  YSCV_REQUIRE(path != nullptr && packed != nullptr && scales != nullptr, "null argument");
  File in;
  in.f = fopen(path, "rb");
  if (!in.f) return set_error(YSCV_HIP_ERR_INVALID_ARG, "cannot open %s: %s", path, strerror(errno));
  yscv_hip_int4_file_header h{};
  Sections s{};
  YSCV_TRY(read_header(in.f, path, &h, &s));
  YSCV_REQUIRE(packed_bytes == s.packed && scales_bytes == s.scales, "%s holds %zu + %zu bytes of nibbles + scales, buffers have %zu + %zu",
               path, s.packed, s.scales, packed_bytes, scales_bytes);
  YSCV_REQUIRE(zero_points_bytes == s.zps && (s.zps == 0 || zero_points != nullptr), "%s holds %zu bytes of zero points, buffer has %zu", path,
               s.zps, zero_points_bytes);
  YSCV_TRY(read_section(in.f, packed, s.packed, "packed nibbles", path));
  YSCV_TRY(read_section(in.f, scales, s.scales, "scales", path));
  if (s.zps) YSCV_TRY(read_section(in.f, zero_points, s.zps, "zero points", path));
  uint64_t sum = fnv1a(kFnvSeed, packed, s.packed);
  sum = fnv1a(sum, scales, s.scales);
  if (s.zps) sum = fnv1a(sum, zero_points, s.zps);
  if (sum != h.checksum)
    return set_error(YSCV_HIP_ERR_INVALID_ARG, "%s: checksum mismatch (stored %016llx, contents %016llx)", path,
                     (unsigned long long)h.checksum, (unsigned long long)sum);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_int4_weight_load(const char *path, yscv_hip_int4_weight **out) {
  YSCV_REQUIRE(path != nullptr && out != nullptr, "null argument");
  yscv_hip_int4_file_header h{};
  YSCV_TRY(yscv_hip_int4_file_read_header(path, &h));
  std::vector<uint8_t> packed, scales, zps;
  try {
    packed.resize(h.packed_bytes);
    scales.resize(h.scales_bytes);
    zps.resize(h.zero_points_bytes);
  } catch (const std::bad_alloc &) {
    return set_error(YSCV_HIP_ERR_OOM, "%s: no host memory for %llu bytes", path,
                     (unsigned long long)(h.packed_bytes + h.scales_bytes + h.zero_points_bytes));
  }
  YSCV_TRY(yscv_hip_int4_file_read(path, packed.data(), packed.size(), scales.data(), scales.size(),
                                   zps.empty() ? nullptr : zps.data(), zps.size()));
  return yscv_hip_int4_weight_create(packed.data(), scales.data(), h.scale_dtype, zps.empty() ? nullptr : zps.data(), h.nibble_format,
                                     (size_t)h.n, (size_t)h.k, (size_t)h.group_size, out);
}

}  // extern "C"
