// .npz reading and writing for TensorFile; see tpuhip/tensor_file.hpp.
#include "tpuhip/tensor_file.hpp"

#include <zlib.h>

#include <cstdio>
#include <cstring>
#include <stdexcept>

namespace tpuhip {

namespace {

[[noreturn]] void fail(const std::string &what) { throw std::runtime_error("TensorFile: " + what); }

uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
uint32_t rd32(const uint8_t *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
uint64_t rd64(const uint8_t *p) { return (uint64_t)rd32(p) | ((uint64_t)rd32(p + 4) << 32); }
void wr16(std::vector<uint8_t> &v, uint16_t x) { v.push_back((uint8_t)x); v.push_back((uint8_t)(x >> 8)); }
void wr32(std::vector<uint8_t> &v, uint32_t x) { for (int i = 0; i < 4; ++i) v.push_back((uint8_t)(x >> (8 * i))); }
void wr64(std::vector<uint8_t> &v, uint64_t x) { for (int i = 0; i < 8; ++i) v.push_back((uint8_t)(x >> (8 * i))); }

constexpr uint32_t kLocalSig = 0x04034b50, kCentralSig = 0x02014b50, kEndSig = 0x06054b50;
constexpr uint32_t kEnd64Sig = 0x06064b50, kEnd64LocSig = 0x07064b50;

// the header dictionary of a .npy member -> dtype, order and shape
NpyArray parse_npy(const uint8_t *p, size_t n, const std::string &member) {
  if (n < 10 || std::memcmp(p, "\x93NUMPY", 6) != 0) fail("member '" + member + "' is not a .npy array");
  const int major = p[6];
  size_t hlen, hoff;
  if (major == 1) { hlen = rd16(p + 8); hoff = 10; }
  else if (major == 2 || major == 3) { if (n < 12) fail("truncated .npy header"); hlen = rd32(p + 8); hoff = 12; }
  else fail("member '" + member + "': .npy version " + std::to_string(major) + " is not supported");
  if (hoff + hlen > n) fail("member '" + member + "': truncated .npy header");
  const std::string h((const char *)p + hoff, hlen);
  NpyArray a;
  auto value_after = [&](const char *key) -> size_t {
    size_t k = h.find(key);
    if (k == std::string::npos) fail("member '" + member + "': no " + key + " in the .npy header");
    k = h.find(':', k);
    if (k == std::string::npos) fail("member '" + member + "': malformed .npy header");
    ++k;
    while (k < h.size() && h[k] == ' ') ++k;
    return k;
  };
  {
    size_t k = value_after("'descr'");
    if (h[k] != '\'' && h[k] != '"') fail("member '" + member + "': structured dtypes are not supported");
    const char q = h[k];
    const size_t e = h.find(q, k + 1);
    const std::string descr = h.substr(k + 1, e - k - 1);
    if (descr.size() < 3) fail("member '" + member + "': dtype '" + descr + "' is not supported");
    if (descr[0] == '>') fail("member '" + member + "': big-endian data is not supported");
    a.kind = descr[1];
    a.word_size = std::atoi(descr.c_str() + 2);
    if (!(a.kind == 'f' || a.kind == 'i' || a.kind == 'u' || a.kind == 'b') || a.word_size < 1 || a.word_size > 8)
      fail("member '" + member + "': dtype '" + descr + "' is not supported");
  }
  {
    size_t k = value_after("'fortran_order'");
    a.fortran_order = h.compare(k, 4, "True") == 0;
  }
  {
    size_t k = value_after("'shape'");
    if (h[k] != '(') fail("member '" + member + "': malformed shape");
    const size_t e = h.find(')', k);
    std::string t = h.substr(k + 1, e - k - 1);
    size_t q = 0;
    while (q < t.size()) {
      while (q < t.size() && (t[q] == ' ' || t[q] == ',')) ++q;
      if (q >= t.size()) break;
      size_t b = q;
      while (q < t.size() && t[q] >= '0' && t[q] <= '9') ++q;
      if (b == q) fail("member '" + member + "': malformed shape");
      a.shape.push_back(std::strtoll(t.substr(b, q - b).c_str(), nullptr, 10));
      while (q < t.size() && t[q] == 'L') ++q;
    }
  }
  const size_t want = a.count() * (size_t)a.word_size;
  if (hoff + hlen + want > n) fail("member '" + member + "': data shorter than its shape says");
  a.bytes.assign(p + hoff + hlen, p + hoff + hlen + want);
  return a;
}

std::vector<uint8_t> npy_header(const NpyArray &a) {
  std::string d = "{'descr': '";
  d += a.word_size == 1 ? '|' : '<';
  d += a.kind;
  d += std::to_string(a.word_size);
  d += "', 'fortran_order': ";
  d += a.fortran_order ? "True" : "False";
  d += ", 'shape': (";
  for (size_t i = 0; i < a.shape.size(); ++i) {
    d += std::to_string(a.shape[i]);
    if (i + 1 < a.shape.size() || a.shape.size() == 1) d += ",";
    if (i + 1 < a.shape.size()) d += " ";
  }
  d += "), }";
  // the data starts at a multiple of 64 bytes; the dictionary ends with a newline
  const size_t unpadded = 10 + d.size() + 1;
  d.append((64 - unpadded % 64) % 64, ' ');
  d += '\n';
  std::vector<uint8_t> h;
  const char magic[] = "\x93NUMPY";
  h.insert(h.end(), magic, magic + 6);
  if (d.size() < 65536) {
    h.push_back(1); h.push_back(0);
    wr16(h, (uint16_t)d.size());
  } else {
    fail("array has too many dimensions for a .npy header");
  }
  h.insert(h.end(), d.begin(), d.end());
  return h;
}

}  // namespace

size_t NpyArray::count() const {
  size_t n = 1;
  for (auto v : shape) n *= (size_t)v;
  return n;
}

TensorFile::TensorFile(const std::string &filename_, bool readOnly_, bool newCreate)
    : filename(filename_), readOnly(readOnly_) {
  if (newCreate) return;
  try {
    load();
  } catch (const std::exception &) {
    if (readOnly) throw;
    map.clear();
  }
  if (readOnly && map.empty()) fail(filename + " not exist, failed to read for read");
}

void TensorFile::load() {
  FILE *f = std::fopen(filename.c_str(), "rb");
  if (!f) fail(filename + " doesn't exist, please check");
  std::vector<uint8_t> buf;
  std::fseek(f, 0, SEEK_END);
  const long sz = std::ftell(f);
  std::fseek(f, 0, SEEK_SET);
  if (sz < 0) { std::fclose(f); fail("cannot size " + filename); }
  buf.resize((size_t)sz);
  const size_t got = sz ? std::fread(buf.data(), 1, (size_t)sz, f) : 0;
  std::fclose(f);
  if (got != (size_t)sz) fail("short read of " + filename);
  if (buf.size() < 22) fail(filename + " is not a zip archive");

  // end of central directory: the last record, possibly followed by a comment
  size_t eocd = std::string::npos;
  for (size_t back = 22; back <= buf.size() && back <= 22 + 65535; ++back) {
    if (rd32(&buf[buf.size() - back]) == kEndSig) { eocd = buf.size() - back; break; }
  }
  if (eocd == std::string::npos) fail(filename + " is not a zip archive (no end record)");
  uint64_t entries = rd16(&buf[eocd + 10]);
  uint64_t cd_off = rd32(&buf[eocd + 16]);
  if ((entries == 0xffff || cd_off == 0xffffffffu) && eocd >= 20 && rd32(&buf[eocd - 20]) == kEnd64LocSig) {
    const uint64_t e64 = rd64(&buf[eocd - 20 + 8]);
    // offsets come from the file: compare against what is left, so that a value near 2^64 cannot wrap
    if (buf.size() < 56 || e64 > buf.size() - 56 || rd32(&buf[e64]) != kEnd64Sig) fail(filename + ": bad zip64 end record");
    entries = rd64(&buf[e64 + 32]);
    cd_off = rd64(&buf[e64 + 48]);
  }
  if (cd_off > buf.size()) fail(filename + ": bad central directory");
  size_t p = (size_t)cd_off;
  for (uint64_t e = 0; e < entries; ++e) {
    if (buf.size() - p < 46 || rd32(&buf[p]) != kCentralSig) fail(filename + ": bad central directory");
    const uint16_t method = rd16(&buf[p + 10]);
    uint64_t csize = rd32(&buf[p + 20]), usize = rd32(&buf[p + 24]);
    const uint16_t nlen = rd16(&buf[p + 28]), xlen = rd16(&buf[p + 30]), clen = rd16(&buf[p + 32]);
    uint64_t lho = rd32(&buf[p + 42]);
    if (buf.size() - p - 46 < (size_t)nlen + xlen + clen) fail(filename + ": truncated central directory");
    std::string member((const char *)&buf[p + 46], nlen);
    // zip64 extra field: the values that are 0xffffffff above, in this order
    size_t x = p + 46 + nlen;
    const size_t xend = x + xlen;
    while (x + 4 <= xend) {
      const uint16_t id = rd16(&buf[x]), len = rd16(&buf[x + 2]);
      if (id == 0x0001) {
        size_t q = x + 4;
        if (usize == 0xffffffffu && q + 8 <= xend) { usize = rd64(&buf[q]); q += 8; }
        if (csize == 0xffffffffu && q + 8 <= xend) { csize = rd64(&buf[q]); q += 8; }
        if (lho == 0xffffffffu && q + 8 <= xend) { lho = rd64(&buf[q]); q += 8; }
      }
      x += 4 + (size_t)len;
    }
    p += 46 + (size_t)nlen + xlen + clen;
    if (buf.size() < 30 || lho > buf.size() - 30 || rd32(&buf[lho]) != kLocalSig) fail(filename + ": bad local header of " + member);
    const size_t data = (size_t)lho + 30 + rd16(&buf[lho + 26]) + rd16(&buf[lho + 28]);
    if (data > buf.size() || csize > buf.size() - data) fail(filename + ": member " + member + " runs past the end of the file");
    std::string name = member;
    if (name.size() > 4 && name.compare(name.size() - 4, 4, ".npy") == 0) name.resize(name.size() - 4);
    if (method == 0) {
      map[name] = parse_npy(&buf[data], (size_t)csize, member);
    } else if (method == 8) {
      if (csize > 0xffffffffu || usize > 0xffffffffu) fail("compressed member " + member + " is too large");
      std::vector<uint8_t> raw((size_t)usize);
      z_stream zs{};
      if (inflateInit2(&zs, -MAX_WBITS) != Z_OK) fail("zlib init failed");
      zs.next_in = &buf[data];
      zs.avail_in = (uInt)csize;
      zs.next_out = raw.data();
      zs.avail_out = (uInt)usize;
      const int rc = inflate(&zs, Z_FINISH);
      inflateEnd(&zs);
      if (rc != Z_STREAM_END) fail(filename + ": cannot inflate " + member);
      map[name] = parse_npy(raw.data(), raw.size(), member);
    } else {
      fail(filename + ": member " + member + " uses compression method " + std::to_string(method));
    }
  }
}

const NpyArray *TensorFile::find(const std::string &name) const {
  auto it = map.find(name);
  return it == map.end() ? nullptr : &it->second;
}

std::vector<std::string> TensorFile::names() const {
  std::vector<std::string> out;
  for (auto &kv : map) out.push_back(kv.first);
  return out;
}

bool TensorFile::addTensor(const std::string &name, const NpyArray &array) {
  if (readOnly) fail("addTensor on a read-only file");
  if (map.count(name)) return false;
  if (array.bytes.size() != array.count() * (size_t)array.word_size) fail("addTensor: byte count does not match the shape");
  map[name] = array;
  ++changes;
  return true;
}

bool TensorFile::addTensor(const std::string &name, const float *data, const std::vector<int64_t> &shape) {
  NpyArray a;
  a.shape = shape;
  a.kind = 'f';
  a.word_size = 4;
  const size_t n = a.count();
  a.bytes.resize(n * 4);
  if (n) std::memcpy(a.bytes.data(), data, n * 4);
  return addTensor(name, a);
}

bool TensorFile::readTensor(const std::string &name, float *data, size_t count) const {
  auto *a = find(name);
  if (!a) return false;
  if (a->kind != 'f' || a->word_size != 4) return false;
  if (a->num_bytes() != count * sizeof(float)) return false;
  if (count) std::memcpy(data, a->bytes.data(), a->num_bytes());
  return true;
}

bool TensorFile::readTensorAsFloat(const std::string &name, std::vector<float> &data, std::vector<int64_t> &shape) const {
  auto *a = find(name);
  if (!a) return false;
  const size_t n = a->count();
  data.resize(n);
  shape = a->shape;
  const uint8_t *p = a->bytes.data();
  for (size_t i = 0; i < n; ++i) {
    const uint8_t *e = p + i * (size_t)a->word_size;
    double v = 0;
    if (a->kind == 'f' && a->word_size == 4) { float f; std::memcpy(&f, e, 4); v = f; }
    else if (a->kind == 'f' && a->word_size == 8) { std::memcpy(&v, e, 8); }
    else if (a->kind == 'b' || (a->kind == 'u' && a->word_size == 1)) v = *e;
    else if (a->kind == 'i' && a->word_size == 1) v = (int8_t)*e;
    else if (a->kind == 'i' && a->word_size == 2) { int16_t t; std::memcpy(&t, e, 2); v = t; }
    else if (a->kind == 'u' && a->word_size == 2) { uint16_t t; std::memcpy(&t, e, 2); v = t; }
    else if (a->kind == 'i' && a->word_size == 4) { int32_t t; std::memcpy(&t, e, 4); v = t; }
    else if (a->kind == 'u' && a->word_size == 4) { uint32_t t; std::memcpy(&t, e, 4); v = t; }
    else if (a->kind == 'i' && a->word_size == 8) { int64_t t; std::memcpy(&t, e, 8); v = (double)t; }
    else if (a->kind == 'u' && a->word_size == 8) { uint64_t t; std::memcpy(&t, e, 8); v = (double)t; }
    else return false;
    data[i] = (float)v;
  }
  if (a->fortran_order && a->shape.size() > 1) return false;
  return true;
}

bool TensorFile::deleteTensor(const std::string &name) {
  if (readOnly) return false;
  auto it = map.find(name);
  if (it == map.end()) return false;
  map.erase(it);
  ++changes;
  return true;
}

void TensorFile::readAllTensors(std::vector<std::string> &names_, std::vector<std::vector<float>> &tensors,
                                std::vector<std::vector<int64_t>> &shapes) const {
  for (auto &kv : map) {
    const NpyArray &a = kv.second;
    if (a.kind != 'f' || a.word_size != 4) fail("readAllTensors: '" + kv.first + "' is not float32 (support float only for now)");
    std::vector<float> t(a.count());
    if (!t.empty()) std::memcpy(t.data(), a.bytes.data(), a.num_bytes());
    tensors.push_back(std::move(t));
    shapes.push_back(a.shape);
    names_.push_back(kv.first);
  }
}

int TensorFile::keep() {
  if (readOnly) fail("keep on a read-only file");
  if (changes == 0) return 0;
  FILE *f = std::fopen(filename.c_str(), "wb");
  if (!f) fail("cannot create " + filename);
  std::vector<uint8_t> central;
  uint64_t offset = 0, count = 0;
  auto put = [&](const void *p, size_t n) {
    if (n && std::fwrite(p, 1, n, f) != n) { std::fclose(f); fail("short write to " + filename); }
    offset += n;
  };
  for (auto &kv : map) {
    const std::string member = kv.first + ".npy";
    const std::vector<uint8_t> head = npy_header(kv.second);
    const uint64_t size = head.size() + kv.second.bytes.size();
    uLong crc = crc32(0L, Z_NULL, 0);
    crc = crc32(crc, head.data(), (uInt)head.size());
    {
      // crc32 takes 32-bit lengths
      const uint8_t *p = kv.second.bytes.data();
      size_t left = kv.second.bytes.size();
      while (left) {
        const size_t n = left > (1u << 30) ? (1u << 30) : left;
        crc = crc32(crc, p, (uInt)n);
        p += n;
        left -= n;
      }
    }
    const bool big = size >= 0xffffffffull || offset >= 0xffffffffull;
    const uint64_t lho = offset;
    std::vector<uint8_t> extra;
    if (big) { wr16(extra, 0x0001); wr16(extra, 16); wr64(extra, size); wr64(extra, size); }
    std::vector<uint8_t> lh;
    wr32(lh, kLocalSig);
    wr16(lh, big ? 45 : 20);
    wr16(lh, 0); wr16(lh, 0); wr16(lh, 0); wr16(lh, 0x21);   // flags, stored, time 0, date 1980-01-01
    wr32(lh, (uint32_t)crc);
    wr32(lh, big ? 0xffffffffu : (uint32_t)size);
    wr32(lh, big ? 0xffffffffu : (uint32_t)size);
    wr16(lh, (uint16_t)member.size());
    wr16(lh, (uint16_t)extra.size());
    put(lh.data(), lh.size());
    put(member.data(), member.size());
    put(extra.data(), extra.size());
    put(head.data(), head.size());
    put(kv.second.bytes.data(), kv.second.bytes.size());

    std::vector<uint8_t> cx;
    if (big) { wr16(cx, 0x0001); wr16(cx, 24); wr64(cx, size); wr64(cx, size); wr64(cx, lho); }
    wr32(central, kCentralSig);
    wr16(central, big ? 45 : 20);
    wr16(central, big ? 45 : 20);
    wr16(central, 0); wr16(central, 0); wr16(central, 0); wr16(central, 0x21);
    wr32(central, (uint32_t)crc);
    wr32(central, big ? 0xffffffffu : (uint32_t)size);
    wr32(central, big ? 0xffffffffu : (uint32_t)size);
    wr16(central, (uint16_t)member.size());
    wr16(central, (uint16_t)cx.size());
    wr16(central, 0); wr16(central, 0); wr16(central, 0);
    wr32(central, 0);
    wr32(central, big ? 0xffffffffu : (uint32_t)lho);
    central.insert(central.end(), member.begin(), member.end());
    central.insert(central.end(), cx.begin(), cx.end());
    ++count;
  }
  const uint64_t cd_off = offset;
  put(central.data(), central.size());
  std::vector<uint8_t> end;
  if (cd_off >= 0xffffffffull || count >= 0xffff || central.size() >= 0xffffffffull) {
    const uint64_t e64 = offset;
    wr32(end, kEnd64Sig); wr64(end, 44); wr16(end, 45); wr16(end, 45); wr32(end, 0); wr32(end, 0);
    wr64(end, count); wr64(end, count); wr64(end, central.size()); wr64(end, cd_off);
    wr32(end, kEnd64LocSig); wr32(end, 0); wr64(end, e64); wr32(end, 1);
  }
  wr32(end, kEndSig); wr16(end, 0); wr16(end, 0);
  wr16(end, count >= 0xffff ? 0xffff : (uint16_t)count);
  wr16(end, count >= 0xffff ? 0xffff : (uint16_t)count);
  wr32(end, central.size() >= 0xffffffffull ? 0xffffffffu : (uint32_t)central.size());
  wr32(end, cd_off >= 0xffffffffull ? 0xffffffffu : (uint32_t)cd_off);
  wr16(end, 0);
  put(end.data(), end.size());
  if (std::fclose(f) != 0) fail("cannot close " + filename);
  const int ret = changes;
  changes = 0;
  return ret;
}

std::unique_ptr<TensorFile> openInputTensorFile(const std::string &filename) {
  return std::make_unique<TensorFile>(filename, true);
}

std::unique_ptr<TensorFile> openOutputTensorFile(const std::string &filename) {
  return std::make_unique<TensorFile>(filename, false, true);
}

}  // namespace tpuhip
