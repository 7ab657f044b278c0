#include "loaders/npz_load.h"

#include <zlib.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <vector>

#include "core/enforce.h"

namespace turbo_transformers {
namespace loaders {

namespace {

struct File {
  std::FILE* f = nullptr;
  explicit File(const std::string& name) : f(std::fopen(name.c_str(), "rb")) {
    TT_ENFORCE(f != nullptr, "cannot open %s", name.c_str());
  }
  ~File() {
    if (f) std::fclose(f);
  }
  void Seek(int64_t off, int whence = SEEK_SET) { TT_ENFORCE_EQ(fseeko(f, off, whence), 0, "seek failed"); }
  int64_t Tell() { return ftello(f); }
  void Read(void* dst, size_t n) { TT_ENFORCE_EQ(std::fread(dst, 1, n, f), n, "unexpected end of file"); }
};

// A member that has been inflated into memory, read like a file.
struct MemReader {
  const unsigned char* p;
  size_t left;
  void Read(void* dst, size_t n) {
    TT_ENFORCE(n <= left, "unexpected end of a compressed member");
    std::memcpy(dst, p, n);
    p += n;
    left -= n;
  }
};

// Raw deflate stream (ZIP method 8) -> `usize` bytes.
std::vector<unsigned char> Inflate(const std::vector<unsigned char>& in, uint64_t usize) {
  std::vector<unsigned char> out(usize);
  z_stream zs;
  std::memset(&zs, 0, sizeof(zs));
  TT_ENFORCE_EQ(inflateInit2(&zs, -MAX_WBITS), Z_OK, "inflateInit2 failed");
  size_t in_pos = 0, out_pos = 0;
  int rc = Z_OK;
  while (rc != Z_STREAM_END) {  // avail_in / avail_out are 32-bit: feed members larger than 4 GiB in pieces
    const size_t in_chunk = std::min<size_t>(in.size() - in_pos, 1u << 30), out_chunk = std::min<size_t>(out.size() - out_pos, 1u << 30);
    zs.next_in = const_cast<unsigned char*>(in.data()) + in_pos;
    zs.avail_in = (uInt)in_chunk;
    zs.next_out = out.data() + out_pos;
    zs.avail_out = (uInt)out_chunk;
    rc = inflate(&zs, Z_NO_FLUSH);
    in_pos += in_chunk - zs.avail_in;
    out_pos += out_chunk - zs.avail_out;
    if (rc != Z_OK && rc != Z_STREAM_END) break;
    if (rc == Z_OK && in_chunk - zs.avail_in == 0 && out_chunk - zs.avail_out == 0) break;  // no progress: truncated
  }
  inflateEnd(&zs);
  TT_ENFORCE(rc == Z_STREAM_END && out_pos == usize, "corrupt compressed member (zlib status %d)", rc);
  return out;
}

template <typename T>
T Get(const unsigned char* p) {
  T v;
  std::memcpy(&v, p, sizeof(T));
  return v;  // ZIP and NPY are little-endian, as is the host
}

// ZIP64 extended information: present when a 32-bit field is 0xFFFFFFFF.
void ApplyZip64(const unsigned char* extra, size_t extra_len, uint64_t* usize, uint64_t* csize, uint64_t* offset) {
  size_t pos = 0;
  while (pos + 4 <= extra_len) {
    const uint16_t id = Get<uint16_t>(extra + pos), len = Get<uint16_t>(extra + pos + 2);
    if (id == 0x0001) {
      size_t q = pos + 4;
      if (usize && *usize == 0xFFFFFFFFull && q + 8 <= pos + 4 + len) { *usize = Get<uint64_t>(extra + q); q += 8; }
      if (csize && *csize == 0xFFFFFFFFull && q + 8 <= pos + 4 + len) { *csize = Get<uint64_t>(extra + q); q += 8; }
      if (offset && *offset == 0xFFFFFFFFull && q + 8 <= pos + 4 + len) { *offset = Get<uint64_t>(extra + q); q += 8; }
      return;
    }
    pos += 4 + len;
  }
}

template <typename Reader>
NpyArray ParseNpy(Reader& file, uint64_t size) {
  unsigned char head[12];
  file.Read(head, 10);
  TT_ENFORCE(std::memcmp(head, "\x93NUMPY", 6) == 0, "not an npy member");
  const int major = head[6];
  size_t header_len;
  size_t consumed = 10;
  if (major == 1) {
    header_len = Get<uint16_t>(head + 8);
  } else {
    file.Read(head + 10, 2);
    header_len = Get<uint32_t>(head + 8);
    consumed = 12;
  }
  TT_ENFORCE(consumed + header_len <= size, "npy header is longer than its member");
  std::string header(header_len, '\0');
  file.Read(&header[0], header_len);
  consumed += header_len;

  NpyArray arr;
  // Every position found in the header text is checked: a malformed member must end in EnforceNotMet, not in
  // std::out_of_range from substr or std::invalid_argument from stoi.
  auto need = [&](size_t pos, const char* what) -> size_t {
    TT_ENFORCE(pos != std::string::npos && pos < header.size(), "malformed npy header (%s)", what);
    return pos;
  };
  auto find_value = [&](const std::string& key) -> size_t {
    const size_t k = header.find("'" + key + "'");
    TT_ENFORCE(k != std::string::npos, "npy header lacks %s", key.c_str());
    return need(header.find(':', k), key.c_str()) + 1;
  };
  size_t p = find_value("descr");
  p = need(header.find('\'', p), "descr");
  const size_t descr_end = need(header.find('\'', p + 1), "descr");
  const std::string descr = header.substr(p + 1, descr_end - p - 1);
  TT_ENFORCE(descr.size() >= 3 && descr.size() <= 4 && (descr[0] == '<' || descr[0] == '|') &&
                 descr.find_first_not_of("0123456789", 2) == std::string::npos,
             "unsupported npy dtype %s", descr.c_str());
  arr.kind = descr[1];
  arr.word_size = std::stoi(descr.substr(2));
  TT_ENFORCE((arr.kind == 'f' && (arr.word_size == 4 || arr.word_size == 2)) || (arr.kind == 'i' && arr.word_size == 8),
             "unsupported npy dtype %s (float32, float16 and int64 are read)", descr.c_str());
  p = find_value("fortran_order");
  p = need(header.find_first_not_of(' ', p), "fortran_order");
  TT_ENFORCE(header.compare(p, 5, "False") == 0, "fortran-ordered arrays are not supported");
  p = find_value("shape");
  const size_t lp = need(header.find('(', p), "shape");
  const size_t rp = need(header.find(')', lp), "shape");
  std::string dims = header.substr(lp + 1, rp - lp - 1);
  size_t q = 0;
  uint64_t numel = 1;
  while (q < dims.size()) {
    while (q < dims.size() && (dims[q] == ' ' || dims[q] == ',')) ++q;
    if (q >= dims.size()) break;
    size_t e = q;
    while (e < dims.size() && dims[e] >= '0' && dims[e] <= '9') ++e;
    TT_ENFORCE(e > q && e - q <= 18, "malformed npy shape");
    const uint64_t dim = std::stoull(dims.substr(q, e - q));
    // the product is bounded by the member's size at every step, so it cannot wrap around
    TT_ENFORCE(dim == 0 || numel <= size / dim, "npy shape is larger than its member");
    numel *= dim;
    arr.shape.push_back((int64_t)dim);
    q = e;
  }
  TT_ENFORCE(numel <= size / (uint64_t)arr.word_size, "npy shape is larger than its member");
  const uint64_t payload = numel * (uint64_t)arr.word_size;
  TT_ENFORCE_EQ(consumed + payload, size, "npy member size does not match its shape");
  arr.bytes.resize(payload);
  if (payload) file.Read(arr.bytes.data(), payload);
  return arr;
}

}  // namespace

std::map<std::string, NpyArray> LoadNpz(const std::string& filename) {
  File file(filename);
  file.Seek(0, SEEK_END);
  const int64_t file_size = file.Tell();
  // End-of-central-directory record: scan the tail for its signature.
  const int64_t tail = std::min<int64_t>(file_size, 65536 + 22 + 20 + 56);
  std::vector<unsigned char> buf(tail);
  file.Seek(file_size - tail);
  file.Read(buf.data(), tail);
  int64_t eocd = -1;
  for (int64_t i = tail - 22; i >= 0; --i)
    if (Get<uint32_t>(buf.data() + i) == 0x06054b50u) { eocd = i; break; }
  TT_ENFORCE(eocd >= 0, "%s is not a zip archive", filename.c_str());
  uint64_t entries = Get<uint16_t>(buf.data() + eocd + 10);
  uint64_t cd_offset = Get<uint32_t>(buf.data() + eocd + 16);
  if (entries == 0xFFFF || cd_offset == 0xFFFFFFFFull) {
    // ZIP64: locator (sig 0x07064b50) sits right before the EOCD and points to the ZIP64 EOCD.
    TT_ENFORCE(eocd >= 20 && Get<uint32_t>(buf.data() + eocd - 20) == 0x07064b50u, "zip64 locator missing");
    const uint64_t z64 = Get<uint64_t>(buf.data() + eocd - 20 + 8);
    unsigned char rec[56];
    file.Seek((int64_t)z64);
    file.Read(rec, 56);
    TT_ENFORCE_EQ(Get<uint32_t>(rec), 0x06064b50u, "zip64 end record missing");
    entries = Get<uint64_t>(rec + 32);
    cd_offset = Get<uint64_t>(rec + 48);
  }

  std::map<std::string, NpyArray> out;
  int64_t pos = (int64_t)cd_offset;
  for (uint64_t e = 0; e < entries; ++e) {
    unsigned char h[46];
    file.Seek(pos);
    file.Read(h, 46);
    TT_ENFORCE_EQ(Get<uint32_t>(h), 0x02014b50u, "bad central directory entry");
    const uint16_t method = Get<uint16_t>(h + 10);
    uint64_t csize = Get<uint32_t>(h + 20), usize = Get<uint32_t>(h + 24), local = Get<uint32_t>(h + 42);
    const uint16_t name_len = Get<uint16_t>(h + 28), extra_len = Get<uint16_t>(h + 30), comment_len = Get<uint16_t>(h + 32);
    std::string name(name_len, '\0');
    file.Read(&name[0], name_len);
    std::vector<unsigned char> extra(extra_len);
    if (extra_len) file.Read(extra.data(), extra_len);
    ApplyZip64(extra.data(), extra_len, &usize, &csize, &local);
    // sizes come from the file: bound them by it before anything is allocated from them (a deflated member expands
    // by at most 1032:1)
    TT_ENFORCE(csize <= (uint64_t)file_size && local <= (uint64_t)file_size && usize / 1032 <= (uint64_t)file_size,
               "%s: member %s has sizes beyond the file", filename.c_str(), name.c_str());
    TT_ENFORCE(method != 0 || usize <= (uint64_t)file_size, "%s: member %s is larger than the file", filename.c_str(), name.c_str());
    pos += 46 + name_len + extra_len + comment_len;
    // numpy.savez stores members (method 0); numpy.savez_compressed, which the reference's converter
    // uses (tools/convert_huggingface_bert_pytorch_to_npz.py:71), deflates them (method 8)
    TT_ENFORCE(method == 0 || method == 8, "%s: member %s uses zip compression method %d (stored and deflate are read)",
               filename.c_str(), name.c_str(), (int)method);
    // Local header: 30 bytes + its own name/extra lengths, then the data.
    unsigned char lh[30];
    file.Seek((int64_t)local);
    file.Read(lh, 30);
    TT_ENFORCE_EQ(Get<uint32_t>(lh), 0x04034b50u, "bad local file header");
    file.Seek((int64_t)local + 30 + Get<uint16_t>(lh + 26) + Get<uint16_t>(lh + 28));
    if (name.size() > 4 && name.compare(name.size() - 4, 4, ".npy") == 0) name.resize(name.size() - 4);
    if (method == 0) {
      out.emplace(name, ParseNpy(file, usize));
    } else {
      std::vector<unsigned char> packed(csize);
      if (csize) file.Read(packed.data(), csize);
      const std::vector<unsigned char> raw = Inflate(packed, usize);
      MemReader mem{raw.data(), raw.size()};
      out.emplace(name, ParseNpy(mem, usize));
    }
  }
  return out;
}

}  // namespace loaders
}  // namespace turbo_transformers
