#include "serialize.h"

#include <ATen/hip/HIPEvent.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <fstream>
#include <future>
#include <set>
#include <sstream>
#include <thread>

#include "abi_util.h"

namespace recis {
namespace serialize {

namespace {

const char* const kInterSep = "^";  // serialize/string_sep.cc:5
const char* const kIntraSep = "@";  // serialize/string_sep.cc:6
const char* const kPart = "/part_";
const char* const kEmptySlice = " ";
const char* const kIdSlot = "id";
const char* const kIndexFile = "index";
const char* const kTensorKeyFile = "tensorkey.json";
const char* const kRankJsonFile = "torch_rank_weights_embs_table_multi_shard.json";

bool file_exists(const std::string& p) {
  struct stat st;
  return ::stat(p.c_str(), &st) == 0;
}

std::string read_file(const std::string& p) {
  std::ifstream f(p, std::ios::binary);
  TORCH_CHECK(f.good(), "[", p, "] not found");
  std::stringstream ss;
  ss << f.rdbuf();
  return ss.str();
}

void write_file_atomically(const std::string& p, const std::string& text) {
  const std::string tmp = p + ".tmp";
  {
    std::ofstream f(tmp, std::ios::binary | std::ios::trunc);
    TORCH_CHECK(f.good(), "cannot write ", tmp);
    f << text;
  }
  TORCH_CHECK(std::rename(tmp.c_str(), p.c_str()) == 0, "cannot rename ", tmp, " to ", p);
}

void make_dirs(const std::string& path) {
  std::string cur;
  for (size_t i = 0; i <= path.size(); ++i) {
    if (i == path.size() || path[i] == '/') {
      if (!cur.empty() && !file_exists(cur)) ::mkdir(cur.c_str(), 0777);
    }
    if (i < path.size()) cur.push_back(path[i]);
  }
}

std::string join(const std::string& dir, const std::string& name) { return dir + "/" + name; }

void wait_for(const std::vector<std::string>& paths, const char* what, double timeout) {
  const auto deadline = std::chrono::steady_clock::now() + std::chrono::duration<double>(timeout);
  for (;;) {
    std::string missing;
    for (const auto& p : paths) {
      if (!file_exists(p)) missing += (missing.empty() ? "" : ", ") + p;
    }
    if (missing.empty()) return;
    TORCH_CHECK(std::chrono::steady_clock::now() <= deadline, "timed out waiting for ", what, " of other shards: ",
                missing);
    std::this_thread::sleep_for(std::chrono::milliseconds(100));
  }
}

bool starts_with(const std::string& s, const std::string& prefix) {
  return s.size() >= prefix.size() && s.compare(0, prefix.size(), prefix) == 0;
}

std::vector<std::string> split(const std::string& s, const std::string& sep) {
  std::vector<std::string> out;
  size_t at = 0;
  for (;;) {
    const size_t next = s.find(sep, at);
    if (next == std::string::npos) {
      out.push_back(s.substr(at));
      return out;
    }
    out.push_back(s.substr(at, next - at));
    at = next + sep.size();
  }
}

std::string replace_all(std::string s, const std::string& from, const std::string& to) {
  for (size_t at = 0; (at = s.find(from, at)) != std::string::npos; at += to.size()) s.replace(at, from.size(), to);
  return s;
}

// ---- JSON text
void dump_string(const std::string& s, std::string* out) {
  out->push_back('"');
  for (unsigned char c : s) {
    switch (c) {
      case '"': *out += "\\\""; break;
      case '\\': *out += "\\\\"; break;
      case '\b': *out += "\\b"; break;
      case '\f': *out += "\\f"; break;
      case '\n': *out += "\\n"; break;
      case '\r': *out += "\\r"; break;
      case '\t': *out += "\\t"; break;
      default:
        if (c < 0x20) {
          char buf[8];
          std::snprintf(buf, sizeof(buf), "\\u%04x", c);
          *out += buf;
        } else {
          out->push_back(static_cast<char>(c));  // UTF-8 passes through
        }
    }
  }
  out->push_back('"');
}

void dump_value(const Json& v, int indent, int depth, std::string* out) {
  auto newline = [&](int d) {
    if (indent >= 0) {
      out->push_back('\n');
      out->append(static_cast<size_t>(indent * d), ' ');
    }
  };
  switch (v.kind) {
    case Json::kNull: *out += "null"; break;
    case Json::kBool: *out += v.b ? "true" : "false"; break;
    case Json::kInt: *out += std::to_string(v.i); break;
    case Json::kDouble: {
      char buf[40];
      std::snprintf(buf, sizeof(buf), "%.17g", v.d);
      *out += buf;
      break;
    }
    case Json::kString: dump_string(v.s, out); break;
    case Json::kArray:
      if (v.arr.empty()) {
        *out += "[]";
        break;
      }
      out->push_back('[');
      for (size_t k = 0; k < v.arr.size(); ++k) {
        if (k) out->push_back(',');
        newline(depth + 1);
        dump_value(v.arr[k], indent, depth + 1, out);
      }
      newline(depth);
      out->push_back(']');
      break;
    case Json::kObject:
      if (v.obj.empty()) {
        *out += "{}";
        break;
      }
      out->push_back('{');
      for (size_t k = 0; k < v.obj.size(); ++k) {
        if (k) out->push_back(',');
        newline(depth + 1);
        dump_string(v.obj[k].first, out);
        *out += indent >= 0 ? ": " : ":";
        dump_value(v.obj[k].second, indent, depth + 1, out);
      }
      newline(depth);
      out->push_back('}');
      break;
  }
}

struct Parser {
  const std::string& t;
  size_t at = 0;
  explicit Parser(const std::string& text) : t(text) {}
  void ws() {
    while (at < t.size() && (t[at] == ' ' || t[at] == '\n' || t[at] == '\t' || t[at] == '\r')) ++at;
  }
  [[noreturn]] void fail(const char* what) { TORCH_CHECK(false, "bad JSON (", what, ") at byte ", at); }
  char peek() {
    ws();
    if (at >= t.size()) fail("unexpected end");
    return t[at];
  }
  void expect(char c) {
    if (peek() != c) fail("unexpected character");
    ++at;
  }
  static void put_utf8(unsigned cp, std::string* out) {
    if (cp < 0x80) {
      out->push_back(static_cast<char>(cp));
    } else if (cp < 0x800) {
      out->push_back(static_cast<char>(0xC0 | (cp >> 6)));
      out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
      out->push_back(static_cast<char>(0xE0 | (cp >> 12)));
      out->push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
      out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    } else {
      out->push_back(static_cast<char>(0xF0 | (cp >> 18)));
      out->push_back(static_cast<char>(0x80 | ((cp >> 12) & 0x3F)));
      out->push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
      out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    }
  }
  unsigned hex4() {
    if (at + 4 > t.size()) fail("short \\u escape");
    unsigned v = 0;
    for (int k = 0; k < 4; ++k) {
      const char c = t[at++];
      v <<= 4;
      if (c >= '0' && c <= '9') v |= c - '0';
      else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
      else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
      else fail("bad \\u escape");
    }
    return v;
  }
  std::string string() {
    expect('"');
    std::string out;
    for (;;) {
      if (at >= t.size()) fail("unterminated string");
      const char c = t[at++];
      if (c == '"') return out;
      if (c != '\\') {
        out.push_back(c);
        continue;
      }
      if (at >= t.size()) fail("unterminated escape");
      const char e = t[at++];
      switch (e) {
        case '"': out.push_back('"'); break;
        case '\\': out.push_back('\\'); break;
        case '/': out.push_back('/'); break;
        case 'b': out.push_back('\b'); break;
        case 'f': out.push_back('\f'); break;
        case 'n': out.push_back('\n'); break;
        case 'r': out.push_back('\r'); break;
        case 't': out.push_back('\t'); break;
        case 'u': {
          unsigned cp = hex4();
          if (cp >= 0xD800 && cp < 0xDC00 && at + 1 < t.size() && t[at] == '\\' && t[at + 1] == 'u') {
            at += 2;
            cp = 0x10000 + ((cp - 0xD800) << 10) + (hex4() - 0xDC00);
          }
          put_utf8(cp, &out);
          break;
        }
        default: fail("bad escape");
      }
    }
  }
  Json value() {
    const char c = peek();
    if (c == '{') {
      ++at;
      Json v = Json::Object();
      if (peek() == '}') {
        ++at;
        return v;
      }
      for (;;) {
        ws();
        std::string key = string();
        expect(':');
        v.obj.emplace_back(std::move(key), value());
        const char n = peek();
        ++at;
        if (n == '}') return v;
        if (n != ',') fail("expected , or }");
      }
    }
    if (c == '[') {
      ++at;
      Json v = Json::Array();
      if (peek() == ']') {
        ++at;
        return v;
      }
      for (;;) {
        v.arr.push_back(value());
        const char n = peek();
        ++at;
        if (n == ']') return v;
        if (n != ',') fail("expected , or ]");
      }
    }
    if (c == '"') return Json::Str(string());
    if (t.compare(at, 4, "true") == 0) {
      at += 4;
      return Json::Bool(true);
    }
    if (t.compare(at, 5, "false") == 0) {
      at += 5;
      return Json::Bool(false);
    }
    if (t.compare(at, 4, "null") == 0) {
      at += 4;
      return Json();
    }
    const size_t beg = at;
    bool real = false;
    while (at < t.size() && (std::isdigit(static_cast<unsigned char>(t[at])) || t[at] == '-' || t[at] == '+' ||
                             t[at] == '.' || t[at] == 'e' || t[at] == 'E')) {
      real = real || t[at] == '.' || t[at] == 'e' || t[at] == 'E';
      ++at;
    }
    if (beg == at) fail("unexpected token");
    const std::string num = t.substr(beg, at - beg);
    Json v;
    if (real) {
      v.kind = Json::kDouble;
      v.d = std::strtod(num.c_str(), nullptr);
    } else {
      v.kind = Json::kInt;
      v.i = std::strtoll(num.c_str(), nullptr, 10);
    }
    return v;
  }
};

}  // namespace

// ------------------------------------------------------------------------------------ Json
Json Json::Bool(bool v) {
  Json j;
  j.kind = kBool;
  j.b = v;
  return j;
}
Json Json::Int(int64_t v) {
  Json j;
  j.kind = kInt;
  j.i = v;
  return j;
}
Json Json::Str(std::string v) {
  Json j;
  j.kind = kString;
  j.s = std::move(v);
  return j;
}
Json Json::Array() {
  Json j;
  j.kind = kArray;
  return j;
}
Json Json::Object() {
  Json j;
  j.kind = kObject;
  return j;
}
Json& Json::Set(const std::string& key, Json v) {
  for (auto& kv : obj) {
    if (kv.first == key) {
      kv.second = std::move(v);
      return kv.second;
    }
  }
  obj.emplace_back(key, std::move(v));
  return obj.back().second;
}
const Json* Json::Find(const std::string& key) const {
  for (const auto& kv : obj) {
    if (kv.first == key) return &kv.second;
  }
  return nullptr;
}
bool Json::Erase(const std::string& key) {
  for (auto it = obj.begin(); it != obj.end(); ++it) {
    if (it->first == key) {
      obj.erase(it);
      return true;
    }
  }
  return false;
}
void Json::SortKeys(bool deep) {
  std::stable_sort(obj.begin(), obj.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
  if (deep) {
    for (auto& kv : obj) kv.second.SortKeys(true);
    for (auto& v : arr) v.SortKeys(true);
  }
}
std::string Json::Dump(int indent) const {
  std::string out;
  dump_value(*this, indent, 0, &out);
  return out;
}
Json Json::Parse(const std::string& text) {
  Parser p(text);
  Json v = p.value();
  p.ws();
  TORCH_CHECK(p.at == text.size(), "bad JSON: trailing text at byte ", p.at);
  return v;
}

// ------------------------------------------------------------------------------------ names
std::string DtypeToString(at::ScalarType dtype) {
  switch (dtype) {
    case at::kBool: return "bool";
    case at::kChar: return "I8";
    case at::kByte: return "U8";
    case at::kShort: return "I16";
    case at::kInt: return "I32";
    case at::kLong: return "I64";
    case at::kHalf: return "F16";
    case at::kBFloat16: return "BF16";
    case at::kFloat: return "F32";
    case at::kDouble: return "F64";
    default: TORCH_CHECK(false, "Dtype: ", dtype, " not supported!");
  }
}

at::ScalarType StringToDtype(const std::string& s) {
  // (the reference writes "bool" but only reads "BOOL": both are read here)
  if (s == "bool" || s == "BOOL") return at::kBool;
  if (s == "I8") return at::kChar;
  if (s == "U8") return at::kByte;
  if (s == "I16") return at::kShort;
  if (s == "I32") return at::kInt;
  if (s == "I64") return at::kLong;
  if (s == "F16") return at::kHalf;
  if (s == "BF16") return at::kBFloat16;
  if (s == "F32") return at::kFloat;
  if (s == "F64") return at::kDouble;
  TORCH_CHECK(false, "dtype: ", s, " is invalid");
}

namespace {
// save_bundle.cc:40-54
std::string type_map(const std::string& s) {
  static const std::map<std::string, std::string> m = {
      {"F64", "float64"}, {"F32", "float32"}, {"F16", "float16"}, {"BF16", "bfloat16"}, {"I64", "int64"},
      {"U64", "uint64"},  {"I32", "int32"},   {"U32", "uint32"},  {"I16", "int16"},     {"U16", "uint16"},
      {"I8", "int8"},     {"U8", "uint8"},    {"BOOL", "bool"}};
  auto it = m.find(s);
  return it == m.end() ? std::string() : it->second;
}

std::string zfill(int64_t v, size_t width) {
  std::string s = std::to_string(v);
  return s.size() >= width ? s : std::string(width - s.size(), '0') + s;
}
}  // namespace

std::string SliceToString(int64_t begin, int64_t end, int64_t size) {
  const size_t width = std::to_string(size).size();
  return zfill(begin, width) + kIntraSep + zfill(end, width) + kIntraSep + std::to_string(size);
}

std::vector<int64_t> SliceFromString(const std::string& msg) {
  auto tokens = split(msg, kIntraSep);
  TORCH_CHECK(tokens.size() == 3, "SliceInfo::FromString failed, msg: ", msg);
  return {std::stoll(tokens[0]), std::stoll(tokens[1]), std::stoll(tokens[2])};
}

// slice_info.h:22-37: same slice_size and overlapping [begin, end) ranges
bool SlicesIntersect(const std::vector<int64_t>& a, const std::vector<int64_t>& b) {
  auto one_way = [](const std::vector<int64_t>& l, const std::vector<int64_t>& r) {
    return (l[0] <= r[0] && r[0] < l[1]) || (l[0] < r[1] && r[1] <= l[1]);
  };
  return a[2] == b[2] && (one_way(a, b) || one_way(b, a));
}

std::string DataFileName(int64_t file_index, int64_t file_count) {
  char buf[64];
  std::snprintf(buf, sizeof(buf), "model-%06lld-of-%06lld.safetensors", static_cast<long long>(file_index),
                static_cast<long long>(file_count));
  return buf;
}

std::string BlockName(const std::string& tensor_name, const std::string& slice_info) {
  return tensor_name + kInterSep + slice_info;
}

namespace {
int64_t env_int(const char* name, int64_t fallback) {
  const char* v = std::getenv(name);
  return v && *v ? std::atoll(v) : fallback;
}
}  // namespace
int64_t BlockWriteSize() { return env_int("RECIS_BLOCK_WRITE_SIZE", 1 << 20); }
int64_t BlockReadSize() { return env_int("RECIS_BLOCK_READ_SIZE", 1 << 20); }

// ------------------------------------------------------------------------------------ write blocks
WriteBlock::WriteBlock(std::string tensor_name, std::string slice_info, bool dense, at::ScalarType dtype,
                       std::vector<int64_t> shape)
    : tensor_name_(std::move(tensor_name)),
      slice_info_(std::move(slice_info)),
      dense_(dense),
      dtype_(dtype),
      shape_(std::move(shape)) {
  nbytes_ = static_cast<int64_t>(c10::elementSize(dtype));
  for (int64_t d : shape_) nbytes_ *= d;
}

std::string WriteBlock::MetaKey() const {
  if (tensor_name_.find(kPart) != std::string::npos) return tensor_name_;
  return BlockName(tensor_name_, slice_info_);
}

namespace {

void write_all(std::FILE* f, const void* data, int64_t n) {
  if (n > 0) TORCH_CHECK(std::fwrite(data, 1, static_cast<size_t>(n), f) == static_cast<size_t>(n), "short write");
}

class HostWriteBlock : public WriteBlock {
 public:
  HostWriteBlock(const std::string& name, const std::string& slice, bool dense, at::Tensor t)
      : WriteBlock(name, slice, dense, t.scalar_type(), t.sizes().vec()), t_(std::move(t)) {}
  int64_t WriteData(std::FILE* file) override {
    write_all(file, t_.data_ptr(), nbytes_);
    return nbytes_;
  }

 private:
  at::Tensor t_;
};

// Rows `index` of one slot (write_block.cc:150-199).
class SlotWriteBlock : public WriteBlock {
 public:
  SlotWriteBlock(const std::string& name, const std::string& slice, at::Tensor index, embedding::SlotPtr slot)
      : WriteBlock(name, slice, false, slot->Dtype(), Shape(index, *slot)), index_(std::move(index)), slot_(std::move(slot)) {}
  int64_t WriteData(std::FILE* file) override {
    const int64_t n = index_.numel(), step = std::max<int64_t>(1, BlockWriteSize());
    if (n == 0) return 0;
    c10::DeviceGuard guard(index_.device());
    std::vector<int64_t> buf_shape = shape_;
    buf_shape[0] = std::min(step, n);
    auto pinned = at::TensorOptions().dtype(dtype_).pinned_memory(true);
    at::Tensor bufs[2] = {at::empty(buf_shape, pinned), at::empty(buf_shape, pinned)};
    at::cuda::CUDAEvent events[2];
    int64_t written = 0;
    int pending = -1;
    int64_t pending_rows = 0;
    const int64_t row_bytes = n ? nbytes_ / n : 0;
    int k = 0;
    for (int64_t beg = 0; beg < n; beg += step, ++k) {
      const int64_t end = std::min(beg + step, n);
      at::Tensor rows = slot_->IndexSelect(index_, beg, end);
      bufs[k & 1].narrow(0, 0, end - beg).copy_(rows, /*non_blocking=*/true);
      events[k & 1].record();
      if (pending >= 0) {
        events[pending].synchronize();
        write_all(file, bufs[pending].data_ptr(), pending_rows * row_bytes);
        written += pending_rows * row_bytes;
      }
      pending = k & 1;
      pending_rows = end - beg;
    }
    events[pending].synchronize();
    write_all(file, bufs[pending].data_ptr(), pending_rows * row_bytes);
    return written + pending_rows * row_bytes;
  }

 private:
  static std::vector<int64_t> Shape(const at::Tensor& index, embedding::Slot& slot) {
    std::vector<int64_t> s{index.numel()};
    auto rs = slot.RowShape();
    s.insert(s.end(), rs.begin(), rs.end());
    return s;
  }
  at::Tensor index_;
  embedding::SlotPtr slot_;
};

}  // namespace

WriteBlockPtr MakeTensorWriteBlock(const std::string& name, const at::Tensor& tensor) {
  return c10::make_intrusive<HostWriteBlock>(name, kEmptySlice, true, tensor.detach().to(at::kCPU).contiguous());
}

WriteBlockPtr MakeArrayWriteBlock(const std::string& name, const std::string& slice_info, const at::Tensor& rows) {
  return c10::make_intrusive<HostWriteBlock>(name, slice_info, false, rows.detach().to(at::kCPU).contiguous());
}

std::vector<WriteBlockPtr> MakeHTWriteBlocks(const HashTablePtr& table) {
  auto map = table->ids_map();
  at::Tensor ids = std::get<0>(map), index = std::get<1>(map);
  auto info = table->ChildrenInfo();
  const std::vector<std::string> children = info->Children();
  std::vector<int64_t> counts;
  if (info->IsCoalesce()) {
    at::Tensor tag = at::bitwise_and(at::bitwise_right_shift(ids, info->IdBitsNum()), (int64_t(1) << info->IndexBitsNum()) - 1);
    at::Tensor order = at::argsort(tag, /*stable=*/true, /*dim=*/0, /*descending=*/false);
    at::Tensor per_child = at::bincount(tag, {}, static_cast<int64_t>(children.size())).to(at::kCPU);
    for (int64_t c = 0; c < per_child.numel(); ++c) counts.push_back(per_child[c].item<int64_t>());
    for (size_t c = children.size(); c < counts.size(); ++c) {
      TORCH_CHECK(counts[c] == 0, "table holds keys tagged for a child it does not have");
    }
    ids = at::bitwise_and(ids, info->IdMask()).index_select(0, order);
    index = index.index_select(0, order);
  } else {
    counts.push_back(ids.numel());
  }
  const auto s = table->SliceInfo();
  const std::string slice_info = SliceToString(s[0], s[1], s[2]);
  at::Tensor ids_host = ids.to(at::kCPU);
  std::vector<WriteBlockPtr> blocks;
  auto slots = table->RawSlotGroup()->Slots();
  int64_t beg = 0;
  for (size_t c = 0; c < children.size(); ++c) {
    const int64_t end = beg + (c < counts.size() ? counts[c] : 0);
    blocks.push_back(c10::make_intrusive<HostWriteBlock>(children[c] + kIntraSep + kIdSlot, slice_info, false,
                                                         ids_host.slice(0, beg, end).contiguous()));
    for (const auto& slot : slots) {
      blocks.push_back(c10::make_intrusive<SlotWriteBlock>(children[c] + kIntraSep + slot->Name(), slice_info,
                                                           index.slice(0, beg, end), slot));
    }
    beg = end;
  }
  return blocks;
}

void WriteDataFile(const std::string& path, const std::string& json_path, const std::vector<WriteBlockPtr>& blocks) {
  Json meta = Json::Object();
  int64_t offset = 0;
  for (const auto& b : blocks) {
    Json entry = Json::Object();
    entry.Set("dtype", Json::Str(DtypeToString(b->Dtype())));
    Json shape = Json::Array();
    for (int64_t d : b->Shape()) shape.arr.push_back(Json::Int(d));
    entry.Set("shape", std::move(shape));
    Json offsets = Json::Array();
    offsets.arr.push_back(Json::Int(offset));
    offsets.arr.push_back(Json::Int(offset + b->NumBytes()));
    entry.Set("data_offsets", std::move(offsets));
    entry.Set("dense", Json::Bool(b->IsDense()));
    meta.Set(b->MetaKey(), std::move(entry));
    offset += b->NumBytes();
  }
  {
    std::ofstream f(json_path, std::ios::binary | std::ios::trunc);
    TORCH_CHECK(f.good(), "cannot write ", json_path);
    f << meta.Dump();
  }
  for (auto& kv : meta.obj) kv.second.Erase("dense");
  std::string header = meta.Dump();
  header.append(8 - header.size() % 8, ' ');
  std::FILE* f = std::fopen(path.c_str(), "wb");
  TORCH_CHECK(f != nullptr, "cannot write ", path);
  std::vector<char> io_buf(8 << 20);
  std::setvbuf(f, io_buf.data(), _IOFBF, io_buf.size());
  try {
    const uint64_t header_size = header.size();
    write_all(f, &header_size, 8);
    write_all(f, header.data(), static_cast<int64_t>(header.size()));
    for (const auto& b : blocks) {
      const int64_t written = b->WriteData(f);
      TORCH_CHECK(written == b->NumBytes(), "block ", b->TensorName(), " wrote ", written, " bytes, header says ",
                  b->NumBytes());
    }
  } catch (...) {
    std::fclose(f);
    throw;
  }
  TORCH_CHECK(std::fclose(f) == 0, "cannot finish ", path);
}

// ------------------------------------------------------------------------------------ SaveBundle
namespace {
// index_info.cc: block name -> file number, file name -> number
std::string index_text(std::vector<std::pair<std::string, int64_t>> block_index,
                       std::vector<std::pair<std::string, int64_t>> file_index) {
  Json out = Json::Object(), blocks = Json::Object(), files = Json::Object();
  std::sort(block_index.begin(), block_index.end());
  std::sort(file_index.begin(), file_index.end());
  for (const auto& kv : block_index) blocks.Set(kv.first, Json::Int(kv.second));
  for (const auto& kv : file_index) files.Set(kv.first, Json::Int(kv.second));
  out.Set("block_index", std::move(blocks));
  out.Set("file_index", std::move(files));
  return out.Dump();
}

void index_append(std::vector<std::pair<std::string, int64_t>>& file_index,
                  std::vector<std::pair<std::string, int64_t>>& block_index, const std::string& name,
                  const std::string& file_name) {
  int64_t number = -1;
  for (const auto& kv : file_index) {
    if (kv.first == file_name) number = kv.second;
  }
  if (number < 0) {
    number = static_cast<int64_t>(file_index.size());
    file_index.emplace_back(file_name, number);
  }
  for (auto& kv : block_index) {
    if (kv.first == name) {
      kv.second = number;
      return;
    }
  }
  block_index.emplace_back(name, number);
}
}  // namespace

SaveBundle::SaveBundle(std::string path, int64_t parallel, int64_t shard_index, int64_t shard_num, double merge_timeout)
    : path_(std::move(path)),
      parallel_(parallel),
      shard_index_(shard_index),
      shard_num_(shard_num),
      merge_timeout_(merge_timeout) {
  TORCH_CHECK(parallel > 0, "parallel must > 0");
  TORCH_CHECK(shard_index >= 0 && shard_num > shard_index, "shard_num must > shard_index");
  writers_.resize(parallel);
  for (int64_t i = 0; i < parallel; ++i) file_names_.push_back(DataFileName(shard_index * parallel + i, parallel * shard_num));
}

std::string SaveBundle::Tmp(const char* kind, int64_t writer, int64_t shard) const {
  char buf[96];
  const std::string k = kind;
  if (k == "data") {
    std::snprintf(buf, sizeof(buf), "ckpt-%07lld-%07lld.data.tmp", (long long)shard, (long long)writer);
  } else if (k == "json") {
    std::snprintf(buf, sizeof(buf), "ckpt-%07lld-%07lld.json.tmp", (long long)shard, (long long)writer);
  } else if (k == "index") {
    std::snprintf(buf, sizeof(buf), "ckpt-%07lld.index", (long long)shard);
  } else {
    std::snprintf(buf, sizeof(buf), "%lldtensorkey.json", (long long)shard);
  }
  return join(path_, buf);
}

void SaveBundle::AddBlock(const WriteBlockPtr& block) {
  const int64_t w = next_;
  next_ = (next_ + 1) % parallel_;
  writers_[w].push_back(block);
  if (!block->IsDense()) {
    const std::string new_name = replace_all(block->TensorName(), kIntraSep, ".") + kPart + std::to_string(shard_index_) +
                                 "_" + std::to_string(shard_num_);
    bool known = false;
    for (const auto& kv : name_map_) known = known || kv.first == new_name;
    if (!known) name_map_.emplace_back(new_name, BlockName(block->TensorName(), block->SliceInfo()));
    block->SetTensorName(new_name);
    index_append(file_index_, block_index_, new_name, file_names_[w]);
  } else {
    index_append(file_index_, block_index_, BlockName(block->TensorName(), block->SliceInfo()), file_names_[w]);
  }
}

// Index first, data files next, the shard's name map last: shard 0 takes the name map of another
// shard as the sign that all of that shard's files are complete.
void SaveBundle::Save() {
  make_dirs(path_);
  write_file_atomically(Tmp("index", 0, shard_index_), index_text(block_index_, file_index_));
  std::vector<std::future<void>> jobs;
  for (int64_t i = 0; i < parallel_; ++i) {
    if (writers_[i].empty()) continue;
    jobs.push_back(std::async(std::launch::async, [this, i]() {
      WriteDataFile(Tmp("data", i, shard_index_), Tmp("json", i, shard_index_), writers_[i]);
    }));
  }
  std::exception_ptr first;
  for (auto& j : jobs) {
    try {
      j.get();
    } catch (...) {
      if (!first) first = std::current_exception();
    }
  }
  if (first) std::rethrow_exception(first);
  for (int64_t i = 0; i < parallel_; ++i) {
    if (writers_[i].empty()) continue;
    const std::string from = Tmp("data", i, shard_index_), to = join(path_, file_names_[i]);
    TORCH_CHECK(std::rename(from.c_str(), to.c_str()) == 0, "cannot rename ", from, " to ", to);
  }
  Json names = Json::Object();
  auto sorted = name_map_;
  std::sort(sorted.begin(), sorted.end());
  for (const auto& kv : sorted) names.Set(kv.first, Json::Str(kv.second));
  write_file_atomically(Tmp("tensorkey", 0, shard_index_), names.Dump(4));
  if (shard_index_ == 0) {
    std::vector<std::string> files;
    for (int64_t s = 0; s < shard_num_; ++s) files.push_back(Tmp("tensorkey", 0, s));
    wait_for(files, "files", merge_timeout_);
    MergeRankJson();
    MergeTensorKeyJson();
  }
}

// save_bundle.cc:277-318. A writer with no blocks leaves no side file.
void SaveBundle::MergeRankJson() {
  std::map<std::string, Json> sub;
  for (int64_t s = 0; s < shard_num_; ++s) {
    for (int64_t w = 0; w < parallel_; ++w) {
      const std::string f = Tmp("json", w, s);
      if (!file_exists(f)) continue;
      Json part = Json::Parse(read_file(f));
      for (auto& kv : part.obj) sub[kv.first] = std::move(kv.second);
      std::remove(f.c_str());
    }
  }
  Json combined = Json::Object();
  for (auto& kv : sub) {  // a std::map: sorted by name
    const std::string& k = kv.first;
    Json v = std::move(kv.second);
    const Json* dense = v.Find("dense");
    const std::string dtype = v.Find("dtype") ? v.Find("dtype")->s : std::string();
    if (dense && dense->b) {
      v.Erase("data_offsets");
      v.Set("name", Json::Str(k));
      v.Set("dtype", Json::Str(type_map(dtype)));
      v.Set("dimension", Json::Int(0));
      v.Set("is_hashmap", Json::Bool(false));
    } else if (k.find(".embedding") != std::string::npos) {
      v.Erase("data_offsets");
      const Json* shape = v.Find("shape");
      const int64_t dim = shape && !shape->arr.empty() ? shape->arr.back().i : 0;
      v.Set("name", Json::Str(k));
      v.Set("dtype", Json::Str(type_map(dtype)));
      v.Set("dimension", Json::Int(dim));
      v.Set("hashmap_key", Json::Str(replace_all(k, ".embedding", ".id")));
      v.Set("hashmap_key_dtype", Json::Str("int64"));
      v.Set("hashmap_value", Json::Str(k));
      v.Set("is_hashmap", Json::Bool(true));
    }
    v.SortKeys(false);
    combined.Set(k, std::move(v));
  }
  std::ofstream f(join(path_, kRankJsonFile), std::ios::binary | std::ios::trunc);
  f << combined.Dump(4);
}

void SaveBundle::MergeTensorKeyJson() {
  std::map<std::string, std::string> combined;
  for (int64_t s = 0; s < shard_num_; ++s) {
    const std::string f = Tmp("tensorkey", 0, s);
    Json part = Json::Parse(read_file(f));
    for (const auto& kv : part.obj) combined[kv.first] = kv.second.s;
    std::remove(f.c_str());
  }
  Json out = Json::Object();
  for (const auto& kv : combined) out.Set(kv.first, Json::Str(kv.second));
  std::ofstream f(join(path_, kTensorKeyFile), std::ios::binary | std::ios::trunc);
  f << out.Dump(4);
}

// save_bundle.cc:124-171: shard 0 folds every shard's index into `index`.
void SaveBundle::MergeMetaInfo() {
  if (shard_index_ != 0) return;
  std::vector<std::string> files;
  for (int64_t s = 0; s < shard_num_; ++s) files.push_back(Tmp("index", 0, s));
  wait_for(files, "indexes", merge_timeout_);
  std::sort(files.begin(), files.end());
  std::vector<std::pair<std::string, int64_t>> file_index, block_index;
  for (const auto& f : files) {
    Json info = Json::Parse(read_file(f));
    const int64_t base = static_cast<int64_t>(file_index.size());
    const Json* fi = info.Find("file_index");
    const Json* bi = info.Find("block_index");
    TORCH_CHECK(fi && bi, "bad index file ", f);
    for (const auto& kv : fi->obj) file_index.emplace_back(kv.first, base + kv.second.i);
    for (const auto& kv : bi->obj) {
      bool replaced = false;
      for (auto& have : block_index) {
        if (have.first == kv.first) {
          have.second = base + kv.second.i;
          replaced = true;
        }
      }
      if (!replaced) block_index.emplace_back(kv.first, base + kv.second.i);
    }
    std::remove(f.c_str());
  }
  write_file_atomically(join(path_, kIndexFile), index_text(block_index, file_index));
}

// ------------------------------------------------------------------------------------ reading
void BlockInfo::ReadInto(void* out, int64_t byte_offset, int64_t nbytes) const {
  if (nbytes == 0) return;
  std::FILE* f = std::fopen(path.c_str(), "rb");
  TORCH_CHECK(f != nullptr, "cannot open ", path);
  std::setvbuf(f, nullptr, _IONBF, 0);
  const bool ok = ::fseeko(f, static_cast<off_t>(offset_beg + byte_offset), SEEK_SET) == 0 &&
                  std::fread(out, 1, static_cast<size_t>(nbytes), f) == static_cast<size_t>(nbytes);
  std::fclose(f);
  TORCH_CHECK(ok, "short read in ", path);
}

at::Tensor BlockInfo::ReadTensor() const {
  at::Tensor t = at::empty(shape, at::TensorOptions().dtype(dtype).device(at::kCPU));
  ReadInto(t.data_ptr(), 0, Size());
  return t;
}

std::vector<std::pair<std::string, BlockInfo>> ReadDataFileHeader(const std::string& path,
                                                                  const std::map<std::string, std::string>* name_map) {
  std::FILE* f = std::fopen(path.c_str(), "rb");
  TORCH_CHECK(f != nullptr, "cannot open ", path);
  uint64_t meta_size = 0;
  std::string text;
  bool ok = std::fread(&meta_size, 1, 8, f) == 8 && meta_size < (uint64_t(1) << 40);
  if (ok) {
    text.resize(meta_size);
    ok = std::fread(&text[0], 1, meta_size, f) == meta_size;
  }
  std::fclose(f);
  TORCH_CHECK(ok, "bad data file header in ", path);
  Json meta = Json::Parse(text);
  const int64_t base = 8 + static_cast<int64_t>(meta_size);
  std::vector<std::pair<std::string, BlockInfo>> out;
  for (const auto& kv : meta.obj) {
    if (kv.first == "__metadata__") continue;
    const Json* dtype = kv.second.Find("dtype");
    const Json* shape = kv.second.Find("shape");
    const Json* offsets = kv.second.Find("data_offsets");
    TORCH_CHECK(dtype && shape && offsets && offsets->arr.size() == 2, "BlockInfo::DecodeFromJson failed, json: ",
                kv.second.Dump());
    BlockInfo b;
    b.dtype = StringToDtype(dtype->s);
    for (const auto& d : shape->arr) b.shape.push_back(d.i);
    b.offset_beg = offsets->arr[0].i + base;
    b.offset_end = offsets->arr[1].i + base;
    b.path = path;
    std::string name = kv.first;
    if (name_map) {
      auto it = name_map->find(name);
      if (it != name_map->end()) name = it->second;
    }
    out.emplace_back(std::move(name), std::move(b));
  }
  return out;
}

LoadBundle::LoadBundle(const std::string& path) : path_(path) {
  Json names = Json::Parse(read_file(join(path, kTensorKeyFile)));
  for (const auto& kv : names.obj) name_map_[kv.first] = kv.second.s;
  const std::string index_file = join(path, kIndexFile);
  TORCH_CHECK(file_exists(index_file), "[", index_file, "] not found");
  Json index = Json::Parse(read_file(index_file));
  const Json* fi = index.Find("file_index");
  const Json* bi = index.Find("block_index");
  TORCH_CHECK(fi && bi, "bad index file ", index_file);
  for (const auto& kv : fi->obj) file_by_number_[kv.second.i] = kv.first;
  for (const auto& kv : bi->obj) {
    auto it = name_map_.find(kv.first);
    block_index_.emplace_back(it == name_map_.end() ? kv.first : it->second, kv.second.i);
  }
}

// index_info.cc:58-66: prefix match on the bare tensor name
bool LoadBundle::HasTensor(const std::string& tensor_name) const {
  for (const auto& kv : block_index_) {
    if (starts_with(kv.first, tensor_name)) return true;
  }
  return false;
}

std::vector<std::string> LoadBundle::ListTensor() const {
  std::set<std::string> names;
  for (const auto& kv : block_index_) {
    auto tokens = split(kv.first, kInterSep);
    TORCH_CHECK(tokens.size() == 2, "block_name: ", kv.first, ", type error");
    names.insert(tokens[0]);
  }
  return std::vector<std::string>(names.begin(), names.end());
}

std::vector<std::string> LoadBundle::SliceInfos(const std::string& tensor_name) const {
  std::vector<std::string> out;
  for (const auto& kv : block_index_) {
    if (!starts_with(kv.first, tensor_name)) continue;
    auto tokens = split(kv.first, kInterSep);
    TORCH_CHECK(tokens.size() == 2, "block_name: ", kv.first, ", type error");
    out.push_back(tokens[1]);
  }
  return out;
}

const BlockInfo& LoadBundle::GetBlockInfo(const std::string& block_name) {
  int64_t number = -1;
  for (const auto& kv : block_index_) {
    if (kv.first == block_name) number = kv.second;
  }
  TORCH_CHECK(number >= 0, "block ", block_name, " not found");
  auto it = headers_.find(number);
  if (it == headers_.end()) {
    std::map<std::string, BlockInfo> header;
    for (auto& kv : ReadDataFileHeader(join(path_, file_by_number_.at(number)), &name_map_)) {
      header[kv.first] = std::move(kv.second);
    }
    it = headers_.emplace(number, std::move(header)).first;
  }
  auto b = it->second.find(block_name);
  TORCH_CHECK(b != it->second.end(), "block ", block_name, " is not in ", file_by_number_.at(number));
  return b->second;
}

std::vector<int64_t> LoadBundle::TensorShape(const std::string& tensor_name) {
  std::vector<int64_t> shape;
  for (const auto& s : SliceInfos(tensor_name)) {
    const BlockInfo& b = GetBlockInfo(BlockName(tensor_name, s));
    if (shape.empty()) {
      shape = b.shape;
    } else {
      shape[0] += b.shape[0];
    }
  }
  return shape;
}

at::ScalarType LoadBundle::TensorType(const std::string& tensor_name) {
  auto slices = SliceInfos(tensor_name);
  TORCH_CHECK(!slices.empty(), tensor_name, " not found");
  return GetBlockInfo(BlockName(tensor_name, slices[0])).dtype;
}

// ------------------------------------------------------------------------------------ Saver
Saver::Saver(int64_t shard_index, int64_t shard_num, int64_t parallel, const std::string& path)
    : parallel_(parallel), shard_index_(shard_index), shard_num_(shard_num), path_(path) {}

// saver.cc:38-54: table blocks of every table, then (shard 0 only) the dense tensors
std::vector<WriteBlockPtr> Saver::MakeWriteBlocks(const c10::Dict<std::string, HashTablePtr>& hashtables,
                                                  const c10::Dict<std::string, at::Tensor>& tensors) {
  std::vector<WriteBlockPtr> blocks;
  for (const auto& kv : hashtables) {
    auto ht_blocks = MakeHTWriteBlocks(kv.value());
    blocks.insert(blocks.end(), ht_blocks.begin(), ht_blocks.end());
  }
  if (shard_index_ == 0) {
    for (const auto& kv : tensors) blocks.push_back(MakeTensorWriteBlock(kv.key(), kv.value()));
  }
  return blocks;
}

void Saver::Save(std::vector<WriteBlockPtr> write_blocks) {
  SaveBundle bundle(path_, parallel_, shard_index_, shard_num_);
  for (const auto& b : write_blocks) bundle.AddBlock(b);
  bundle.Save();
  bundle.MergeMetaInfo();
  if (at::hasHIP() || at::hasCUDA()) {
    // a row index the gathers had to skip means a checkpoint with holes
    int bits = 0;
    recis::hipabi::check(recis_hip_poll_device_errors(&bits));
    TORCH_CHECK(bits == 0, "librecis_hip: device-side errors in earlier kernels (bits ", bits, ")");
  }
}

// ------------------------------------------------------------------------------------ Loader
Loader::Loader(const std::string& path, int64_t parallel, c10::Dict<std::string, HashTablePtr> hts_to_load,
               c10::Dict<std::string, at::Tensor> tensors_to_load)
    : parallel_(parallel), path_(path) {
  for (const auto& kv : hts_to_load) hts_.emplace_back(kv.key(), kv.value());
  for (const auto& kv : tensors_to_load) tensors_.emplace_back(kv.key(), kv.value());
}

std::string Loader::DefaultLoadInfo() {
  Json info = Json::Object();
  for (const auto& ht : hts_) {
    Json slots = Json::Array();
    slots.arr.push_back(Json::Str(kIdSlot));
    for (const auto& s : ht.second->RawSlotGroup()->Slots()) slots.arr.push_back(Json::Str(s->Name()));
    for (const auto& child : ht.second->ChildrenInfo()->Children()) {
      Json entry = Json::Object();
      entry.Set(child, slots);
      if (info.Find(child) == nullptr) {
        info.Set(child, std::move(entry));
      } else {
        for (auto& kv : info.obj) {
          if (kv.first == child) kv.second.Set(child, slots);
        }
      }
    }
  }
  for (const auto& t : tensors_) {
    if (info.Find(t.first) == nullptr) info.Set(t.first, Json::Object());
    for (auto& kv : info.obj) {
      if (kv.first == t.first) kv.second.Set(t.first, Json::Array());
    }
  }
  return info.Dump();
}

namespace {

// read_block.cc:52-65: a key belongs to this table when (uint64)key % slice_size is in [begin, end)
at::Tensor accept_mask(const at::Tensor& ids, const std::vector<int64_t>& s) {
  const int64_t n = ids.numel();
  at::Tensor mask = at::empty({n}, at::TensorOptions().dtype(at::kBool));
  const int64_t* p = ids.data_ptr<int64_t>();
  bool* m = mask.data_ptr<bool>();
  const uint64_t size = static_cast<uint64_t>(s[2]);
  for (int64_t i = 0; i < n; ++i) {
    const int64_t mod = static_cast<int64_t>(static_cast<uint64_t>(p[i]) % size);
    m[i] = mod >= s[0] && mod < s[1];
  }
  return mask;
}

struct Piece {
  embedding::SlotPtr slot;
  const BlockInfo* block;
  int64_t beg, end;
};

// One (child, slice) group: keys first, then every slot in pieces of RECIS_BLOCK_READ_SIZE rows
// (read_block.cc:67-79,94-109,125-163). File reads run on `parallel` threads into a ring of pinned
// buffers; this thread copies each piece to the device and scatters it into the slot, in order.
void load_table_blocks(const HashTablePtr& ht, const std::string& child, const BlockInfo& id_block,
                       const std::vector<std::pair<embedding::SlotPtr, const BlockInfo*>>& slot_blocks,
                       int64_t parallel) {
  at::Tensor ids = id_block.ReadTensor().reshape({-1});
  TORCH_CHECK(ids.scalar_type() == at::kLong, "the id block of ", child, " is not int64");
  at::Tensor accept = accept_mask(ids, ht->SliceInfo());
  auto info = ht->ChildrenInfo();
  if (info->IsCoalesce()) {
    at::Tensor tagged = at::bitwise_or(at::bitwise_and(ids, info->IdMask()),
                                       static_cast<int64_t>(static_cast<uint64_t>(info->ChildIndex(child)) << info->IdBitsNum()));
    ids = at::where(accept, tagged, ids);
  }
  const at::Device device = ht->device();
  c10::DeviceGuard guard(device);
  at::Tensor accept_dev = accept.to(device);
  at::Tensor index = ht->InsertLookupIndexWithIndicator(ids.to(device), accept_dev);
  const int64_t step = std::max<int64_t>(1, BlockReadSize());
  std::vector<Piece> pieces;
  for (const auto& sb : slot_blocks) {
    std::vector<int64_t> want{sb.second->shape.empty() ? 0 : sb.second->shape[0]};
    auto rs = sb.first->RowShape();
    want.insert(want.end(), rs.begin(), rs.end());
    TORCH_CHECK(want == sb.second->shape, "shape not match");
    TORCH_CHECK(sb.first->Dtype() == sb.second->dtype, "dtype not match");
    for (int64_t beg = 0; beg < want[0]; beg += step) pieces.push_back({sb.first, sb.second, beg, std::min(beg + step, want[0])});
  }
  if (pieces.empty()) return;
  const int64_t n_pieces = static_cast<int64_t>(pieces.size());
  const int64_t ring = std::max<int64_t>(2, std::min(parallel, n_pieces) + 1);
  int64_t biggest = 0;
  for (const auto& p : pieces) biggest = std::max(biggest, (p.end - p.beg) * p.block->RowBytes());
  std::vector<at::Tensor> bufs;
  for (int64_t r = 0; r < ring; ++r) {
    bufs.push_back(at::empty({std::max<int64_t>(biggest, 1)}, at::TensorOptions().dtype(at::kByte).pinned_memory(true)));
  }
  std::vector<std::unique_ptr<at::cuda::CUDAEvent>> done(ring);
  auto read = [&](int64_t k) {
    const Piece& p = pieces[k];
    const int64_t row_bytes = p.block->RowBytes();
    if (done[k % ring]) done[k % ring]->synchronize();  // the copy that last used this buffer has finished
    p.block->ReadInto(bufs[k % ring].data_ptr(), p.beg * row_bytes, (p.end - p.beg) * row_bytes);
  };
  std::vector<std::future<void>> futures(n_pieces);
  int64_t issued = 0;
  for (int64_t k = 0; k < n_pieces; ++k) {
    while (issued < n_pieces && issued < k + ring - 1) {
      futures[issued] = std::async(std::launch::async, read, issued);
      ++issued;
    }
    futures[k].get();
    const Piece& p = pieces[k];
    std::vector<int64_t> shape = p.block->shape;
    shape[0] = p.end - p.beg;
    const int64_t nbytes = (p.end - p.beg) * p.block->RowBytes();
    at::Tensor rows = bufs[k % ring].narrow(0, 0, nbytes).to(device, /*non_blocking=*/true).view(p.block->dtype).reshape(shape);
    done[k % ring] = std::make_unique<at::cuda::CUDAEvent>();
    done[k % ring]->record();
    p.slot->IndexInsert(index.slice(0, p.beg, p.end), rows, accept_dev.slice(0, p.beg, p.end));
  }
  for (auto& e : done) {
    if (e) e->synchronize();
  }
}

}  // namespace

void Loader::Load(std::string load_info) {
  Json info = Json::Parse(load_info);
  LoadBundle bundle(path_);
  std::map<std::string, HashTablePtr> name_to_ht;
  for (const auto& ht : hts_) {
    for (const auto& child : ht.second->ChildrenInfo()->Children()) name_to_ht[child] = ht.second;
  }
  // load_internal.cc:96-146
  for (const auto& dst : info.obj) {
    auto found = name_to_ht.find(dst.first);
    if (found == name_to_ht.end()) continue;
    const HashTablePtr& ht = found->second;
    const std::vector<int64_t> mine = ht->SliceInfo();
    for (const auto& src : dst.second.obj) {
      struct Group {
        const BlockInfo* id = nullptr;
        std::vector<std::pair<embedding::SlotPtr, const BlockInfo*>> slots;
      };
      std::vector<std::pair<std::string, Group>> groups;  // by slice string, in order of first appearance
      for (const auto& slot_name_json : src.second.arr) {
        const std::string& slot_name = slot_name_json.s;
        const std::string tensor_name = dst.first + kIntraSep + slot_name;
        if (!bundle.HasTensor(tensor_name)) continue;
        for (const auto& slice_str : bundle.SliceInfos(tensor_name)) {
          if (!SlicesIntersect(SliceFromString(slice_str), mine)) continue;
          Group* g = nullptr;
          for (auto& have : groups) {
            if (have.first == slice_str) g = &have.second;
          }
          if (g == nullptr) {
            groups.emplace_back(slice_str, Group());
            g = &groups.back().second;
          }
          const BlockInfo* b = &bundle.GetBlockInfo(BlockName(tensor_name, slice_str));
          if (slot_name == kIdSlot) {
            g->id = b;
          } else {
            g->slots.emplace_back(ht->RawSlotGroup()->GetSlotByName(slot_name), b);
          }
        }
      }
      for (const auto& g : groups) {
        TORCH_CHECK(g.second.id != nullptr && !g.second.slots.empty(), src.first, ", invalid");
        load_table_blocks(ht, src.first, *g.second.id, g.second.slots, parallel_);
      }
    }
  }
  // load_internal.cc:149-175
  for (const auto& dst : info.obj) {
    at::Tensor target;
    for (const auto& t : tensors_) {
      if (t.first == dst.first) target = t.second;
    }
    if (!target.defined()) continue;
    TORCH_CHECK(dst.second.obj.size() == 1, "currently only support one tensor");
    for (const auto& src : dst.second.obj) {
      if (!bundle.HasTensor(src.first)) continue;
      const BlockInfo& b = bundle.GetBlockInfo(BlockName(src.first, kEmptySlice));
      TORCH_CHECK(b.dtype == target.scalar_type(), "dtype not match");
      TORCH_CHECK(b.shape == target.sizes().vec(), "shape not match");
      c10::NoGradGuard no_grad;
      target.copy_(b.ReadTensor());
    }
  }
  if (at::hasHIP() || at::hasCUDA()) {
    // rows the inserts had to skip would be missing silently
    int bits = 0;
    recis::hipabi::check(recis_hip_poll_device_errors(&bits));
    TORCH_CHECK(bits == 0, "librecis_hip: device-side errors in earlier kernels (bits ", bits, ")");
  }
}

// ------------------------------------------------------------------------------------ CheckpointReader
void CheckpointReader::Init() { bundle_ = c10::make_intrusive<LoadBundle>(path_); }

LoadBundle& CheckpointReader::Bundle() {
  if (!bundle_.defined()) Init();
  return *bundle_;
}

std::vector<std::string> CheckpointReader::ListTensors() { return Bundle().ListTensor(); }

at::Tensor CheckpointReader::LoadTensor(const std::string& tensor_name) {
  TORCH_CHECK(Bundle().HasTensor(tensor_name), tensor_name, " not found");
  auto slices = Bundle().SliceInfos(tensor_name);
  std::sort(slices.begin(), slices.end());
  std::vector<at::Tensor> parts;
  for (const auto& s : slices) parts.push_back(Bundle().GetBlockInfo(BlockName(tensor_name, s)).ReadTensor());
  return parts.size() == 1 ? parts[0] : at::cat(parts, 0);
}

std::vector<int64_t> CheckpointReader::TensorShape(const std::string& tensor_name) {
  TORCH_CHECK(Bundle().HasTensor(tensor_name), tensor_name, " not found");
  return Bundle().TensorShape(tensor_name);
}

at::Tensor CheckpointReader::TensorType(const std::string& tensor_name) {
  TORCH_CHECK(Bundle().HasTensor(tensor_name), tensor_name, " not found");
  return at::empty({}, at::TensorOptions().dtype(Bundle().TensorType(tensor_name)).device(at::kCPU));
}

}  // namespace serialize
}  // namespace recis
