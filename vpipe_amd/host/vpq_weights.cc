// Reader and writer of the quantized checkpoint container (see vpq_weights.h).
#include "vpq_weights.h"

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdio>
#include <cstring>

#include "../../include/vpq.h"

namespace vpipe_amd {

namespace {

// ------------------------------------------------------------------ a small JSON reader
// Enough for a safetensors header and the shard index: objects, arrays, strings, integers.
struct Json {
  enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
  bool b = false;
  double num = 0.0;
  std::int64_t inum = 0;
  bool integral = false;
  std::string str;
  std::vector<Json> items;
  std::vector<std::pair<std::string, Json>> members;

  const Json* get(const char* key) const
  {
    for (const auto& m : members) {
      if (m.first == key) { return &m.second; }
    }
    return nullptr;
  }
};

class JsonParser {
public:
  JsonParser(const char* p, std::size_t n) : _p(p), _end(p + n) {}
  bool parse(Json* out)
  {
    if (!value(out, 0)) { return false; }
    skip();
    return _p == _end;
  }

private:
  static constexpr int kMaxDepth = 16;
  void skip()
  {
    while (_p < _end && (*_p == ' ' || *_p == '\n' || *_p == '\t' || *_p == '\r')) { ++_p; }
  }
  bool literal(const char* s)
  {
    const std::size_t n = std::strlen(s);
    if ((std::size_t)(_end - _p) < n || std::memcmp(_p, s, n) != 0) { return false; }
    _p += n;
    return true;
  }
  static void append_utf8(std::string* s, unsigned cp)
  {
    if (cp < 0x80) {
      s->push_back((char)cp);
    } else if (cp < 0x800) {
      s->push_back((char)(0xC0 | (cp >> 6)));
      s->push_back((char)(0x80 | (cp & 0x3F)));
    } else {
      s->push_back((char)(0xE0 | (cp >> 12)));
      s->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      s->push_back((char)(0x80 | (cp & 0x3F)));
    }
  }
  bool string(std::string* out)
  {
    if (_p >= _end || *_p != '"') { return false; }
    ++_p;
    out->clear();
    while (_p < _end) {
      const char c = *_p++;
      if (c == '"') { return true; }
      if (c != '\\') {
        out->push_back(c);
        continue;
      }
      if (_p >= _end) { return false; }
      const char e = *_p++;
      switch (e) {
        case '"': out->push_back('"'); break;
        case '\\': out->push_back('\\'); break;
        case '/': out->push_back('/'); break;
        case 'b': out->push_back('\b'); break;
        case 'f': out->push_back('\f'); break;
        case 'n': out->push_back('\n'); break;
        case 'r': out->push_back('\r'); break;
        case 't': out->push_back('\t'); break;
        case 'u': {
          if (_end - _p < 4) { return false; }
          unsigned cp = 0;
          for (int i = 0; i < 4; ++i) {
            const char h = *_p++;
            cp <<= 4;
            if (h >= '0' && h <= '9') { cp |= (unsigned)(h - '0'); }
            else if (h >= 'a' && h <= 'f') { cp |= (unsigned)(h - 'a' + 10); }
            else if (h >= 'A' && h <= 'F') { cp |= (unsigned)(h - 'A' + 10); }
            else { return false; }
          }
          append_utf8(out, cp);
          break;
        }
        default: return false;
      }
    }
    return false;
  }
  bool number(Json* out)
  {
    const char* s = _p;
    if (_p < _end && *_p == '-') { ++_p; }
    bool integral = true;
    while (_p < _end && ((*_p >= '0' && *_p <= '9') || *_p == '.' || *_p == 'e' || *_p == 'E' || *_p == '+' || *_p == '-')) {
      if (*_p < '0' || *_p > '9') { integral = false; }
      ++_p;
    }
    if (_p == s || (_p - s) > 40) { return false; }
    const std::string t(s, _p);
    out->kind = Json::Number;
    out->integral = integral;
    errno = 0;
    if (integral) {
      out->inum = std::strtoll(t.c_str(), nullptr, 10);
      out->num = (double)out->inum;
    } else {
      out->num = std::strtod(t.c_str(), nullptr);
    }
    return errno == 0;
  }
  bool value(Json* out, int depth)
  {
    if (depth > kMaxDepth) { return false; }
    skip();
    if (_p >= _end) { return false; }
    const char c = *_p;
    if (c == '{') {
      ++_p;
      out->kind = Json::Object;
      skip();
      if (_p < _end && *_p == '}') { ++_p; return true; }
      for (;;) {
        skip();
        std::string key;
        if (!string(&key)) { return false; }
        skip();
        if (_p >= _end || *_p++ != ':') { return false; }
        Json v;
        if (!value(&v, depth + 1)) { return false; }
        out->members.emplace_back(std::move(key), std::move(v));
        skip();
        if (_p >= _end) { return false; }
        if (*_p == ',') { ++_p; continue; }
        if (*_p == '}') { ++_p; return true; }
        return false;
      }
    }
    if (c == '[') {
      ++_p;
      out->kind = Json::Array;
      skip();
      if (_p < _end && *_p == ']') { ++_p; return true; }
      for (;;) {
        Json v;
        if (!value(&v, depth + 1)) { return false; }
        out->items.push_back(std::move(v));
        skip();
        if (_p >= _end) { return false; }
        if (*_p == ',') { ++_p; continue; }
        if (*_p == ']') { ++_p; return true; }
        return false;
      }
    }
    if (c == '"') {
      out->kind = Json::String;
      return string(&out->str);
    }
    if (c == 't') { out->kind = Json::Bool; out->b = true; return literal("true"); }
    if (c == 'f') { out->kind = Json::Bool; out->b = false; return literal("false"); }
    if (c == 'n') { out->kind = Json::Null; return literal("null"); }
    return number(out);
  }
  const char* _p;
  const char* _end;
};

void json_escape(const std::string& in, std::string* out)
{
  for (const char ch : in) {
    const unsigned char c = (unsigned char)ch;
    if (c == '"' || c == '\\') {
      out->push_back('\\');
      out->push_back(ch);
    } else if (c < 0x20) {
      char buf[8];
      std::snprintf(buf, sizeof(buf), "\\u%04x", c);
      *out += buf;
    } else {
      out->push_back(ch);
    }
  }
}

// Bytes per element of the dtypes a checkpoint of this family holds; 0 = not checked.
int dtype_size(const std::string& d)
{
  if (d == "U8" || d == "I8" || d == "BOOL" || d == "F8_E4M3" || d == "F8_E5M2") { return 1; }
  if (d == "F16" || d == "BF16" || d == "I16" || d == "U16") { return 2; }
  if (d == "F32" || d == "I32" || d == "U32") { return 4; }
  if (d == "F64" || d == "I64" || d == "U64") { return 8; }
  return 0;
}

void set_why(std::string* why, const std::string& text)
{
  if (why != nullptr) { *why = text; }
}

bool pread_all(int fd, void* dst, std::uint64_t n, std::uint64_t at)
{
  std::uint8_t* p = static_cast<std::uint8_t*>(dst);
  while (n > 0) {
    const std::size_t want = (std::size_t)std::min<std::uint64_t>(n, 1ull << 30);
    const ssize_t r = ::pread(fd, p, want, (off_t)at);
    if (r <= 0) { return false; }
    p += r;
    at += (std::uint64_t)r;
    n -= (std::uint64_t)r;
  }
  return true;
}

bool write_all(int fd, const void* src, std::uint64_t n)
{
  const std::uint8_t* p = static_cast<const std::uint8_t*>(src);
  while (n > 0) {
    const std::size_t want = (std::size_t)std::min<std::uint64_t>(n, 1ull << 30);
    const ssize_t w = ::write(fd, p, want);
    if (w <= 0) { return false; }
    p += w;
    n -= (std::uint64_t)w;
  }
  return true;
}

std::string join_path(const std::string& dir, const std::string& name)
{
  if (dir.empty()) { return name; }
  return dir.back() == '/' ? dir + name : dir + "/" + name;
}

bool file_exists(const std::string& p)
{
  struct stat st;
  return ::stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

bool make_dirs(const std::string& dir)
{
  if (dir.empty()) { return true; }
  std::string cur;
  for (std::size_t i = 0; i <= dir.size(); ++i) {
    if (i == dir.size() || dir[i] == '/') {
      if (!cur.empty() && ::mkdir(cur.c_str(), 0755) != 0 && errno != EEXIST) { return false; }
    }
    if (i < dir.size()) { cur.push_back(dir[i]); }
  }
  return true;
}

}  // namespace

// ================================================================== PackFile
PackFile::PackFile(PackFile&& o) noexcept : _shards(std::move(o._shards)), _tensors(std::move(o._tensors))
{
  o._shards.clear();
}

PackFile& PackFile::operator=(PackFile&& o) noexcept
{
  if (this != &o) {
    release();
    _shards = std::move(o._shards);
    _tensors = std::move(o._tensors);
    o._shards.clear();
  }
  return *this;
}

PackFile::~PackFile() { release(); }

void PackFile::release()
{
  for (Shard& s : _shards) {
    if (s.fd >= 0) { ::close(s.fd); }
    s.fd = -1;
  }
  _shards.clear();
  _tensors.clear();
}

bool PackFile::add_shard(const std::string& path, std::string* why)
{
  Shard sh;
  sh.path = path;
  sh.fd = ::open(path.c_str(), O_RDONLY);
  if (sh.fd < 0) {
    set_why(why, path + ": cannot open");
    return false;
  }
  const int index = (int)_shards.size();
  _shards.push_back(sh);           // from here on release() closes the descriptor
  Shard& s = _shards.back();
  struct stat st;
  if (::fstat(s.fd, &st) != 0) {
    set_why(why, path + ": cannot stat");
    return false;
  }
  s.file_size = (std::uint64_t)st.st_size;
  std::uint64_t header_len = 0;
  if (s.file_size < 8 || !pread_all(s.fd, &header_len, 8, 0)) {
    set_why(why, path + ": shorter than its length prefix");
    return false;
  }
  if (header_len < 2 || header_len > (100ull << 20) || 8 + header_len > s.file_size) {
    set_why(why, path + ": header length outside the file");
    return false;
  }
  std::string header((std::size_t)header_len, '\0');
  if (!pread_all(s.fd, &header[0], header_len, 8)) {
    set_why(why, path + ": short read of the header");
    return false;
  }
  Json root;
  if (!JsonParser(header.data(), header.size()).parse(&root) || root.kind != Json::Object) {
    set_why(why, path + ": header is not a JSON object");
    return false;
  }
  s.data_start = 8 + header_len;
  const std::uint64_t blob = s.file_size - s.data_start;
  for (const auto& m : root.members) {
    if (m.first == "__metadata__") { continue; }
    const Json& e = m.second;
    const Json* dt = e.get("dtype");
    const Json* shp = e.get("shape");
    const Json* off = e.get("data_offsets");
    if (e.kind != Json::Object || dt == nullptr || dt->kind != Json::String || shp == nullptr ||
        shp->kind != Json::Array || off == nullptr || off->kind != Json::Array || off->items.size() != 2) {
      set_why(why, path + ": malformed entry '" + m.first + "'");
      return false;
    }
    TensorInfo ti;
    ti.dtype = dt->str;
    ti.shard = index;
    std::uint64_t count = 1;
    for (const Json& d : shp->items) {
      if (d.kind != Json::Number || !d.integral || d.inum < 0) {
        set_why(why, path + ": bad shape of '" + m.first + "'");
        return false;
      }
      ti.shape.push_back(d.inum);
      // keeps the element count below 2^56, so that count * element size cannot wrap
      if (d.inum != 0 && count > ((std::uint64_t)1 << 56) / (std::uint64_t)d.inum) {
        set_why(why, path + ": shape of '" + m.first + "' too large");
        return false;
      }
      count *= (std::uint64_t)d.inum;
    }
    const Json& b0 = off->items[0];
    const Json& b1 = off->items[1];
    if (b0.kind != Json::Number || b1.kind != Json::Number || !b0.integral || !b1.integral || b0.inum < 0 ||
        b1.inum < b0.inum || (std::uint64_t)b1.inum > blob) {
      set_why(why, path + ": byte range of '" + m.first + "' outside the file");
      return false;
    }
    ti.offset = (std::uint64_t)b0.inum;
    ti.nbytes = (std::uint64_t)(b1.inum - b0.inum);
    const int esz = dtype_size(ti.dtype);
    if (esz > 0 && count * (std::uint64_t)esz != ti.nbytes) {
      set_why(why, path + ": '" + m.first + "' has " + std::to_string(ti.nbytes) + " bytes, its dtype and shape say " +
                       std::to_string(count * (std::uint64_t)esz));
      return false;
    }
    _tensors[m.first] = std::move(ti);   // a later shard wins, as a merged namespace does
  }
  return true;
}

std::optional<PackFile> PackFile::open(const std::string& path, std::string* why)
{
  PackFile f;
  if (!f.add_shard(path, why)) { return std::nullopt; }
  return std::optional<PackFile>(std::move(f));
}

std::optional<PackFile> PackFile::open_model(const std::string& dir, std::string* why)
{
  const std::string index_path = join_path(dir, "model.safetensors.index.json");
  if (!file_exists(index_path)) {
    const std::string single = join_path(dir, "model.safetensors");
    if (!file_exists(single)) {
      set_why(why, dir + ": neither model.safetensors.index.json nor model.safetensors");
      return std::nullopt;
    }
    return open(single, why);
  }
  const int fd = ::open(index_path.c_str(), O_RDONLY);
  if (fd < 0) {
    set_why(why, index_path + ": cannot open");
    return std::nullopt;
  }
  struct stat st;
  std::string text;
  bool ok = ::fstat(fd, &st) == 0 && st.st_size > 0 && st.st_size < (256ll << 20);
  if (ok) {
    text.resize((std::size_t)st.st_size);
    ok = pread_all(fd, &text[0], (std::uint64_t)st.st_size, 0);
  }
  ::close(fd);
  Json root;
  if (!ok || !JsonParser(text.data(), text.size()).parse(&root) || root.kind != Json::Object) {
    set_why(why, index_path + ": not a JSON object");
    return std::nullopt;
  }
  const Json* map = root.get("weight_map");
  if (map == nullptr || map->kind != Json::Object) {
    set_why(why, index_path + ": no weight_map");
    return std::nullopt;
  }
  std::vector<std::string> files;      // distinct shard files, in first-mention order
  for (const auto& m : map->members) {
    if (m.second.kind != Json::String) {
      set_why(why, index_path + ": weight_map value of '" + m.first + "' is not a file name");
      return std::nullopt;
    }
    if (std::find(files.begin(), files.end(), m.second.str) == files.end()) { files.push_back(m.second.str); }
  }
  PackFile f;
  for (const std::string& name : files) {
    if (name.find('/') != std::string::npos || name.find("..") != std::string::npos) {
      set_why(why, index_path + ": shard name '" + name + "' leaves the model directory");
      return std::nullopt;
    }
    if (!f.add_shard(join_path(dir, name), why)) { return std::nullopt; }
  }
  // Every tensor the index names must be where it says.
  for (const auto& m : map->members) {
    const TensorInfo* ti = f.info(m.first);
    if (ti == nullptr || f._shards[(std::size_t)ti->shard].path != join_path(dir, m.second.str)) {
      set_why(why, index_path + ": '" + m.first + "' is not in " + m.second.str);
      return std::nullopt;
    }
  }
  return std::optional<PackFile>(std::move(f));
}

const TensorInfo* PackFile::info(const std::string& name) const
{
  const auto it = _tensors.find(name);
  return it == _tensors.end() ? nullptr : &it->second;
}

std::vector<std::string> PackFile::tensor_names() const
{
  std::vector<std::string> out;
  out.reserve(_tensors.size());
  for (const auto& kv : _tensors) { out.push_back(kv.first); }
  return out;
}

PackFile::Alignment PackFile::alignment() const
{
  Alignment a;
  a.shards = (int)_shards.size();
  for (const Shard& s : _shards) {
    if (s.data_start % 16 != 0) { ++a.bad_shards; }
  }
  for (const auto& kv : _tensors) {
    ++a.tensors;
    const Shard& s = _shards[(std::size_t)kv.second.shard];
    if ((s.data_start + kv.second.offset) % 16 != 0) { ++a.misaligned; }
  }
  return a;
}

bool PackFile::read_into(const std::string& name, void* dst, std::size_t capacity) const
{
  const TensorInfo* ti = info(name);
  if (ti == nullptr || dst == nullptr || capacity < ti->nbytes) { return false; }
  const Shard& s = _shards[(std::size_t)ti->shard];
  return ti->nbytes == 0 || pread_all(s.fd, dst, ti->nbytes, s.data_start + ti->offset);
}

int PackFile::affine_bits(const std::string& prefix, int K) const
{
  const TensorInfo* w = info(prefix + ".weight");
  if (w == nullptr || !has(prefix + ".scales") || w->shape.empty() || K <= 0) { return 0; }
  return (int)(w->shape.back() * 32 / K);
}

int PackFile::affine_group(const std::string& prefix, int K) const
{
  const TensorInfo* s = info(prefix + ".scales");
  if (s == nullptr || s->shape.empty() || s->shape.back() <= 0 || K <= 0) { return 0; }
  return (int)(K / s->shape.back());
}

bool PackFile::load_linear(CommandStream& stream, const std::string& prefix, int K, LoadedLinear* out,
                           std::string* why) const
{
  if (out == nullptr || !stream.valid()) {
    set_why(why, "load_linear: no stream or no destination");
    return false;
  }
  const TensorInfo* w = info(prefix + ".weight");
  const TensorInfo* s = info(prefix + ".scales");
  const TensorInfo* b = info(prefix + ".biases");
  if (w == nullptr || s == nullptr || b == nullptr) {
    set_why(why, prefix + ": .weight / .scales / .biases not all present");
    return false;
  }
  if (w->dtype != "U32" || w->shape.size() != 2 || s->shape.size() != 2 || b->shape != s->shape ||
      b->dtype != s->dtype || (s->dtype != "F16" && s->dtype != "BF16")) {
    set_why(why, prefix + ": not a U32 [N, K*bits/32] weight with F16 or BF16 [N, K/group] scales and biases");
    return false;
  }
  if (K <= 0) {
    // No K given: the (width, group) pair that both shapes agree on, among the served ones; K from it.  The shapes
    // alone cannot tell 4-bit group-32 from 8-bit group-64 (same words and same scales per row), so a caller with
    // such packs passes K.
    const long long words = w->shape[1], groups = s->shape[1];
    int found = 0;
    const int cand[2][2] = {{4, 64}, {8, 64}};
    for (const auto& c : cand) {
      const long long k = words * 32 / c[0];
      if (words * 32 % c[0] == 0 && k % c[1] == 0 && k / c[1] == groups && k <= 0x7fffffffLL) {
        K = (int)k;
        ++found;
      }
    }
    if (found != 1) {
      set_why(why, prefix + ": cannot tell the width and group from a [N, " + std::to_string(words) + "] weight with [N, " +
                       std::to_string(groups) + "] scales; pass K");
      return false;
    }
  }
  const int N = (int)w->shape[0];
  // Width and group from the shapes (generative-models/qwen3/metal-qwen-model.cc:653-676); served: 4-bit group-64,
  // 8-bit group-64, 4-bit group-32, 8-bit group-32.
  const int bits = affine_bits(prefix, K), group = affine_group(prefix, K);
  const bool served = (bits == 4 || bits == 8) && (group == 64 || group == 32);
  if (!served || K % group != 0 || w->shape[1] * 32 != (long long)K * bits || s->shape[0] != N ||
      s->shape[1] * group != K) {
    set_why(why, prefix + ": " + std::to_string(bits) + "-bit group-" + std::to_string(group) +
                     " pack; this path takes 4- and 8-bit codes in groups of 64 and 32");
    return false;
  }
  std::vector<std::uint8_t> host((std::size_t)std::max(w->nbytes, s->nbytes));
  LoadedLinear l;
  l.K = K;
  l.N = N;
  l.bits = bits;
  l.group = group;
  l.codes = DeviceBuffer::allocate((std::size_t)w->nbytes);
  l.scales = DeviceBuffer::allocate((std::size_t)s->nbytes);
  l.qbias = DeviceBuffer::allocate((std::size_t)b->nbytes);
  if (l.codes.empty() || l.scales.empty() || l.qbias.empty()) {
    set_why(why, prefix + ": device allocation failed");
    return false;
  }
  if (!read_into(prefix + ".weight", host.data(), host.size()) || !l.codes.upload(host.data(), (std::size_t)w->nbytes)) {
    set_why(why, prefix + ".weight: read or upload failed");
    return false;
  }
  const bool f16 = s->dtype == "F16";
  DeviceBuffer raw;
  if (f16) {
    raw = DeviceBuffer::allocate((std::size_t)s->nbytes);
    if (raw.empty()) {
      set_why(why, prefix + ": device allocation failed");
      return false;
    }
  }
  const char* parts[2] = {".scales", ".biases"};
  DeviceBuffer* dst[2] = {&l.scales, &l.qbias};
  for (int i = 0; i < 2; ++i) {
    if (!read_into(prefix + parts[i], host.data(), host.size())) {
      set_why(why, prefix + parts[i] + ": read failed");
      return false;
    }
    if (!f16) {
      if (!dst[i]->upload(host.data(), (std::size_t)s->nbytes)) {
        set_why(why, prefix + parts[i] + ": upload failed");
        return false;
      }
      continue;
    }
    // F16 on disk, bf16 in the kernels: converted once here (docs/PLUGINS.md:210-213).
    if (!raw.upload(host.data(), (std::size_t)s->nbytes)) {
      set_why(why, prefix + parts[i] + ": upload failed");
      return false;
    }
    const int st = vpq_f16_to_bf16(stream.native(), static_cast<const uint16_t*>(raw.data()),
                                   static_cast<uint16_t*>(dst[i]->data()), (size_t)(s->nbytes / 2));
    if (st != VPQ_OK) { stream.record_error(st, "vpq_f16_to_bf16"); }
    std::string reason;
    if (!stream.commit().wait_ok(&reason)) {   // `raw` is reused for the biases and freed below
      set_why(why, prefix + parts[i] + ": " + reason);
      return false;
    }
  }
  *out = std::move(l);
  return true;
}

// ================================================================== PackWriter
PackWriter::PackWriter(std::string out_dir, std::uint64_t shard_max_bytes)
    : _dir(std::move(out_dir)), _shard_max(shard_max_bytes)
{
  make_dirs(_dir);
}

PackWriter::~PackWriter()
{
  for (Shard& s : _shards) {
    if (s.fd >= 0) { ::close(s.fd); }
    if (!s.blob_path.empty()) { ::unlink(s.blob_path.c_str()); }   // gone already if the shard was finished
  }
}

// Makes sure _shards.back() is open and has room for `incoming` bytes: a non-empty shard that
// would pass the budget is closed first (one oversized tensor still gets a shard to itself).
bool PackWriter::current_shard(std::uint64_t incoming)
{
  if (!_shards.empty()) {
    Shard& cur = _shards.back();
    const std::uint64_t filled = cur.size + cur.held_bytes;
    if (cur.fd >= 0 && (filled == 0 || filled + incoming <= _shard_max)) { return true; }
    if (cur.fd >= 0) {
      ::close(cur.fd);
      cur.fd = -1;
    }
  }
  Shard s;
  s.blob_path = join_path(_dir, ".blob-" + std::to_string(_shards.size()) + ".tmp");
  s.fd = ::open(s.blob_path.c_str(), O_RDWR | O_CREAT | O_TRUNC, 0644);
  if (s.fd < 0) { return false; }
  _shards.push_back(std::move(s));
  return true;
}

bool PackWriter::add(const std::string& name, const std::string& dtype, const std::vector<std::int64_t>& shape,
                     const void* data, std::uint64_t nbytes)
{
  if (_closed || name.empty() || _names.count(name) != 0 || (data == nullptr && nbytes != 0)) { return false; }
  if (!current_shard(nbytes)) { return false; }
  Shard& cur = _shards.back();
  Entry e;
  e.name = name;
  e.dtype = dtype;
  e.shape = shape;
  e.nbytes = nbytes;
  _names[name] = (int)_shards.size() - 1;
  // Tensors tile the blob without gaps, so one whose size is not a multiple of 16 would push
  // every later tensor off the 16-byte boundary: small ones wait in memory and go last.
  if (nbytes % 16 != 0 && nbytes <= kHeldMax && cur.held_bytes + nbytes <= kHeldTotalMax) {
    Held h;
    h.e = std::move(e);
    const std::uint8_t* p = static_cast<const std::uint8_t*>(data);
    h.bytes.assign(p, p + nbytes);
    cur.held_bytes += nbytes;
    cur.held.push_back(std::move(h));
    return true;
  }
  e.offset = cur.size;
  if (!write_all(cur.fd, data, nbytes)) { return false; }
  cur.size += nbytes;
  cur.entries.push_back(std::move(e));
  return true;
}

bool PackWriter::finish_shard(std::size_t idx, std::size_t total, std::string* file_name)
{
  Shard& s = _shards[idx];
  if (!s.held.empty()) {
    if (s.fd < 0) { s.fd = ::open(s.blob_path.c_str(), O_WRONLY | O_APPEND); }
    if (s.fd < 0) { return false; }
    for (Held& h : s.held) {
      h.e.offset = s.size;
      if (!write_all(s.fd, h.bytes.data(), h.bytes.size())) { return false; }
      s.size += h.e.nbytes;
      s.entries.push_back(std::move(h.e));
    }
    s.held.clear();
    s.held_bytes = 0;
  }
  if (s.fd >= 0) {
    ::close(s.fd);
    s.fd = -1;
  }

  std::string header = "{";
  for (std::size_t i = 0; i < s.entries.size(); ++i) {
    const Entry& e = s.entries[i];
    if (i != 0) { header += ","; }
    header += "\"";
    json_escape(e.name, &header);
    header += "\":{\"dtype\":\"";
    json_escape(e.dtype, &header);
    header += "\",\"shape\":[";
    for (std::size_t d = 0; d < e.shape.size(); ++d) {
      if (d != 0) { header += ","; }
      header += std::to_string(e.shape[d]);
    }
    header += "],\"data_offsets\":[" + std::to_string(e.offset) + "," + std::to_string(e.offset + e.nbytes) + "]}";
  }
  header += "}";
  // The blob starts at 8 + header length; trailing spaces (insignificant in JSON, and readers
  // take the length from the prefix) bring that to a multiple of 16.
  header.append((16 - (8 + header.size()) % 16) % 16, ' ');

  char name[64];
  std::snprintf(name, sizeof(name), "model-%05zu-of-%05zu.safetensors", idx + 1, total);
  *file_name = name;
  const std::string final_path = join_path(_dir, name);
  const int out = ::open(final_path.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644);
  if (out < 0) { return false; }
  const std::uint64_t hlen = header.size();
  bool ok = write_all(out, &hlen, 8) && write_all(out, header.data(), header.size());
  if (ok && s.size > 0) {
    const int in = ::open(s.blob_path.c_str(), O_RDONLY);
    ok = in >= 0;
    if (ok) {
      std::vector<std::uint8_t> buf(8u << 20);
      std::uint64_t left = s.size, at = 0;
      while (ok && left > 0) {
        const std::uint64_t n = std::min<std::uint64_t>(left, buf.size());
        ok = pread_all(in, buf.data(), n, at) && write_all(out, buf.data(), n);
        at += n;
        left -= n;
      }
      ::close(in);
    }
  }
  ok = (::close(out) == 0) && ok;
  ::unlink(s.blob_path.c_str());
  s.blob_path.clear();
  return ok;
}

bool PackWriter::close()
{
  if (_closed) { return true; }
  _closed = true;
  if (_shards.empty()) { return true; }
  std::string index = "\"weight_map\":{";
  std::uint64_t total_bytes = 0;
  bool first = true;
  for (std::size_t i = 0; i < _shards.size(); ++i) {
    std::string file;
    if (!finish_shard(i, _shards.size(), &file)) { return false; }
    _files.push_back(file);
    for (const Entry& e : _shards[i].entries) {
      if (!first) { index += ","; }
      first = false;
      index += "\"";
      json_escape(e.name, &index);
      index += "\":\"" + file + "\"";
      total_bytes += e.nbytes;
    }
  }
  index = "{\"metadata\":{\"total_size\":" + std::to_string(total_bytes) + "}," + index + "}}";
  const std::string path = join_path(_dir, "model.safetensors.index.json");
  const int fd = ::open(path.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644);
  if (fd < 0) { return false; }
  const bool ok = write_all(fd, index.data(), index.size());
  return (::close(fd) == 0) && ok;
}

// ================================================================== quantize_and_add
bool quantize_and_add(CommandStream& stream, PackWriter& writer, const std::string& prefix,
                      const DeviceBuffer& src_bf16, int K, int N, float clip, std::string* why)
{
  if (!stream.valid() || src_bf16.empty() || K <= 0 || N <= 0 || K % 64 != 0 ||
      src_bf16.size() < (std::size_t)N * (std::size_t)K * 2) {
    set_why(why, prefix + ": quantize_and_add needs a bf16 [N,K] source with K % 64 == 0");
    return false;
  }
  const std::size_t wbytes = vpq_weight_bytes(N, K), sbytes = vpq_scale_bytes(N, K);
  DeviceBuffer codes = DeviceBuffer::allocate(wbytes), scales = DeviceBuffer::allocate(sbytes),
               biases = DeviceBuffer::allocate(sbytes);
  if (codes.empty() || scales.empty() || biases.empty()) {
    set_why(why, prefix + ": device allocation failed");
    return false;
  }
  const int st = vpq_quantize_w4g64(stream.native(), static_cast<const uint16_t*>(src_bf16.data()),
                                    static_cast<uint32_t*>(codes.data()), static_cast<uint16_t*>(scales.data()),
                                    static_cast<uint16_t*>(biases.data()), K, N, clip);
  if (st != VPQ_OK) { stream.record_error(st, "vpq_quantize_w4g64"); }
  std::string reason;
  if (!stream.commit().wait_ok(&reason)) {
    set_why(why, prefix + ": " + reason);
    return false;
  }
  std::vector<std::uint8_t> host(std::max(wbytes, sbytes));
  const std::vector<std::int64_t> wshape = {N, K / 8}, sshape = {N, K / 64};
  if (!codes.download(host.data(), wbytes) || !writer.add(prefix + ".weight", "U32", wshape, host.data(), wbytes) ||
      !scales.download(host.data(), sbytes) || !writer.add(prefix + ".scales", "F16", sshape, host.data(), sbytes) ||
      !biases.download(host.data(), sbytes) || !writer.add(prefix + ".biases", "F16", sshape, host.data(), sbytes)) {
    set_why(why, prefix + ": download or write failed");
    return false;
  }
  return true;
}

}  // namespace vpipe_amd
