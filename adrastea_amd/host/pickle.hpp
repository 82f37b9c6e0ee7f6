// Reader of PyTorch checkpoints, the step before the u8 weight path: a memory-mapped zip archive
// whose `data.pkl` member is a pickle of the state dict and whose `data/<key>` members hold the
// raw tensor storages.  Host-side mirror of adrastea_models/src/pickle.rs:33-338 (MappedBuffer,
// TensorDataType, PickledTensor, PickledModel::load_file, ShardedModel::load_huggingface,
// load_tensor).  The reference delegates the two file formats to third-party crates that are
// not part of its tree (zip 0.6, a serde-pickle fork, memmap2; Cargo.lock); here both are read
// directly from their published specifications:
//   * zip: end-of-central-directory record (with the zip64 locator for archives beyond 4 GiB),
//     central directory entries, local headers; members must be STORED (pickle.rs:240-242);
//   * pickle: the protocol-2 opcode subset torch.save emits.  Nothing is executed: GLOBAL yields
//     a symbolic name, REDUCE a node holding callable and arguments, and only
//     torch._utils._rebuild_tensor_v2 / collections.OrderedDict are interpreted.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstring>
#include <algorithm>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace adrastea {

// pickle.rs:33-51
class MappedBuffer {
 public:
  explicit MappedBuffer(const std::string& path) {
    fd_ = ::open(path.c_str(), O_RDONLY);
    if (fd_ < 0) throw std::runtime_error("cannot open " + path);
    struct stat st;
    if (fstat(fd_, &st) != 0) { ::close(fd_); throw std::runtime_error("cannot stat " + path); }
    size_ = (size_t)st.st_size;
    if (size_ == 0) { ::close(fd_); throw std::runtime_error(path + " is empty"); }
    void* p = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
    if (p == MAP_FAILED) { ::close(fd_); throw std::runtime_error("cannot map " + path); }
    data_ = (const uint8_t*)p;
  }
  ~MappedBuffer() {
    if (data_) munmap((void*)data_, size_);
    if (fd_ >= 0) ::close(fd_);
  }
  MappedBuffer(const MappedBuffer&) = delete;
  MappedBuffer& operator=(const MappedBuffer&) = delete;
  const uint8_t* data() const { return data_; }
  size_t size() const { return size_; }

 private:
  int fd_ = -1;
  const uint8_t* data_ = nullptr;
  size_t size_ = 0;
};

// pickle.rs:101-120
enum class TensorDataType { I8, I64, F16, F32, F64 };
inline size_t element_size(TensorDataType t) {
  switch (t) {
    case TensorDataType::I8: return 1;
    case TensorDataType::F16: return 2;
    case TensorDataType::F32: return 4;
    default: return 8;
  }
}

// pickle.rs:122-128: byte range [begin, end) of the mapped file
struct PickledTensor {
  TensorDataType dtype;
  std::vector<size_t> shape, stride;
  size_t begin, end;
};

// ---- zip -------------------------------------------------------------------------------------

struct ZipMember {
  size_t data_start, size;
};

namespace detail {

inline uint16_t rd16(const uint8_t* p) { return (uint16_t)(p[0] | p[1] << 8); }
inline uint32_t rd32(const uint8_t* p) { return (uint32_t)rd16(p) | (uint32_t)rd16(p + 2) << 16; }
inline uint64_t rd64(const uint8_t* p) { return (uint64_t)rd32(p) | (uint64_t)rd32(p + 4) << 32; }

// Members of the archive keyed by the LAST path component, as pickle.rs:243-249 keys them.
inline std::map<std::string, ZipMember> read_zip_directory(const uint8_t* d, size_t n) {
  if (n < 22) throw std::runtime_error("not a zip archive");
  // end-of-central-directory record: signature 0x06054b50, within the last 64 KiB + 22 bytes
  size_t eocd = SIZE_MAX;
  for (size_t back = 22; back <= n && back <= 22 + 65535; back++) {
    if (rd32(d + n - back) == 0x06054b50u) { eocd = n - back; break; }
  }
  if (eocd == SIZE_MAX) throw std::runtime_error("zip: end of central directory not found");
  uint64_t entries = rd16(d + eocd + 10), cd_size = rd32(d + eocd + 12), cd_off = rd32(d + eocd + 16);
  if (entries == 0xFFFF || cd_size == 0xFFFFFFFFu || cd_off == 0xFFFFFFFFu) {
    // zip64: locator (0x07064b50) sits right before the record and points at the zip64 record
    if (eocd < 20 || rd32(d + eocd - 20) != 0x07064b50u) throw std::runtime_error("zip64 locator missing");
    const uint64_t rec = rd64(d + eocd - 20 + 8);
    if (n < 56 || rec > n - 56 || rd32(d + rec) != 0x06064b50u) throw std::runtime_error("zip64 record missing");
    entries = rd64(d + rec + 32);
    cd_size = rd64(d + rec + 40);
    cd_off = rd64(d + rec + 48);
  }
  // (every bound below is written as a subtraction: the fields come from the file, and a sum of
  // two 64-bit values chosen by the file can wrap)
  if (cd_off > n || cd_size > n - cd_off) throw std::runtime_error("zip: central directory out of range");
  std::map<std::string, ZipMember> out;
  size_t p = cd_off;
  for (uint64_t i = 0; i < entries; i++) {
    if (p > n || n - p < 46 || rd32(d + p) != 0x02014b50u) throw std::runtime_error("zip: bad central entry");
    const uint16_t method = rd16(d + p + 10);
    uint64_t csize = rd32(d + p + 20), usize = rd32(d + p + 24), lho = rd32(d + p + 42);
    const uint16_t nlen = rd16(d + p + 28), xlen = rd16(d + p + 30), clen = rd16(d + p + 32);
    if (n - p - 46 < (size_t)nlen + xlen + clen) throw std::runtime_error("zip: truncated central entry");
    const std::string name((const char*)d + p + 46, nlen);
    // zip64 extended information (header id 1): the fields that were 0xFFFFFFFF, in this order
    const uint8_t* x = d + p + 46 + nlen;
    for (size_t q = 0; q + 4 <= xlen;) {
      const uint16_t id = rd16(x + q), len = rd16(x + q + 2);
      if (id == 1) {
        // each 8-byte field must lie inside this extra field and inside the extra area
        const size_t lim = std::min((size_t)xlen, q + 4 + (size_t)len);
        size_t o = q + 4;
        auto field = [&](uint64_t& v) {
          if (o + 8 > lim) throw std::runtime_error("zip64: truncated extended information");
          v = rd64(x + o);
          o += 8;
        };
        if (usize == 0xFFFFFFFFu) field(usize);
        if (csize == 0xFFFFFFFFu) field(csize);
        if (lho == 0xFFFFFFFFu) field(lho);
      }
      q += 4 + (size_t)len;
    }
    if (method != 0) throw std::runtime_error("pytorch archives should not contain compressed files");
    if (n < 30 || lho > n - 30 || rd32(d + lho) != 0x04034b50u) throw std::runtime_error("zip: bad local header");
    const size_t start = lho + 30 + rd16(d + lho + 26) + rd16(d + lho + 28);
    if (start > n || usize > n - start) throw std::runtime_error("zip: member out of range");
    const size_t slash = name.find_last_of('/');
    const std::string base = slash == std::string::npos ? name : name.substr(slash + 1);
    if (!base.empty()) out[base] = ZipMember{start, (size_t)usize};
    p += 46 + (size_t)nlen + xlen + clen;
  }
  return out;
}

// ---- pickle ----------------------------------------------------------------------------------

struct Value;
using ValuePtr = std::shared_ptr<Value>;
struct Value {
  enum Kind { None, Bool, Int, Float, Str, Tuple, List, Dict, Global, PersId, Reduce, Mark } kind = None;
  int64_t i = 0;
  double f = 0;
  std::string s;                                   // Str; Global: "module name"
  std::vector<ValuePtr> items;                     // Tuple / List; PersId: [id]; Reduce: [callable, args]
  std::vector<std::pair<ValuePtr, ValuePtr>> dict; // Dict, in insertion order
};
inline ValuePtr mk(Value::Kind k) { auto v = std::make_shared<Value>(); v->kind = k; return v; }

class Unpickler {
 public:
  Unpickler(const uint8_t* d, size_t n) : d_(d), n_(n) {}
  ValuePtr load() {
    for (;;) {
      const uint8_t op = u8();
      switch (op) {
        case 0x80: u8(); break;                                   // PROTO
        case 0x95: take(8); break;                                // FRAME
        case '.': return pop();                                   // STOP
        case '}': push(mk(Value::Dict)); break;                   // EMPTY_DICT
        case ']': push(mk(Value::List)); break;                   // EMPTY_LIST
        case ')': push(mk(Value::Tuple)); break;                  // EMPTY_TUPLE
        case '(': push(mk(Value::Mark)); break;                   // MARK
        case 'N': push(mk(Value::None)); break;
        case 0x88: case 0x89: { auto v = mk(Value::Bool); v->i = op == 0x88; push(v); break; }
        case 'K': { auto v = mk(Value::Int); v->i = u8(); push(v); break; }               // BININT1
        case 'M': { auto v = mk(Value::Int); v->i = rd16(take(2)); push(v); break; }      // BININT2
        case 'J': { auto v = mk(Value::Int); v->i = (int32_t)rd32(take(4)); push(v); break; }  // BININT
        case 0x8a: {                                                                      // LONG1
          const size_t len = u8();
          if (len > 8) throw std::runtime_error("pickle: integer beyond 64 bits");
          const uint8_t* p = take(len);
          uint64_t u = 0;
          for (size_t k = 0; k < len; k++) u |= (uint64_t)p[k] << (8 * k);
          if (len && len < 8 && (p[len - 1] & 0x80)) u |= ~0ull << (8 * len);
          auto v = mk(Value::Int); v->i = (int64_t)u; push(v); break;
        }
        case 'G': {                                                                       // BINFLOAT
          const uint8_t* p = take(8);
          uint64_t u = 0;
          for (int k = 0; k < 8; k++) u = u << 8 | p[k];
          auto v = mk(Value::Float); std::memcpy(&v->f, &u, 8); push(v); break;
        }
        case 'X': str(rd32(take(4))); break;                      // BINUNICODE
        case 0x8c: str(u8()); break;                              // SHORT_BINUNICODE
        case 'U': str(u8()); break;                               // SHORT_BINSTRING
        case 'T': str(rd32(take(4))); break;                      // BINSTRING
        case 'c': {                                               // GLOBAL module\nname\n
          auto v = mk(Value::Global);
          v->s = line() + " ";
          v->s += line();
          push(v); break;
        }
        case 0x93: {                                              // STACK_GLOBAL
          auto name = pop(), module = pop();
          auto v = mk(Value::Global); v->s = module->s + " " + name->s; push(v); break;
        }
        case 'q': memo_[u8()] = top(); break;                     // BINPUT
        case 'r': memo_[rd32(take(4))] = top(); break;            // LONG_BINPUT
        case 0x94: memo_[(uint32_t)memo_.size()] = top(); break;  // MEMOIZE
        case 'h': push(get(u8())); break;                         // BINGET
        case 'j': push(get(rd32(take(4)))); break;                // LONG_BINGET
        case 't': { auto v = mk(Value::Tuple); v->items = pop_to_mark(); push(v); break; }  // TUPLE
        case 0x85: case 0x86: case 0x87: {                        // TUPLE1..3
          auto v = mk(Value::Tuple);
          const int cnt = op - 0x84;
          v->items.resize(cnt);
          for (int k = cnt - 1; k >= 0; k--) v->items[k] = pop();
          push(v); break;
        }
        case 'a': { auto x = pop(); top()->items.push_back(x); break; }                    // APPEND
        case 'e': { auto xs = pop_to_mark(); for (auto& x : xs) top()->items.push_back(x); break; }
        case 's': { auto v = pop(), k = pop(); top()->dict.emplace_back(k, v); break; }    // SETITEM
        case 'u': {                                                                        // SETITEMS
          auto xs = pop_to_mark();
          if (xs.size() % 2) throw std::runtime_error("pickle: odd SETITEMS");
          for (size_t k = 0; k < xs.size(); k += 2) top()->dict.emplace_back(xs[k], xs[k + 1]);
          break;
        }
        case 'Q': { auto v = mk(Value::PersId); v->items.push_back(pop()); push(v); break; }  // BINPERSID
        case 'R': case 0x81: {                                    // REDUCE / NEWOBJ: never called
          auto args = pop(), callable = pop();
          if (callable->kind == Value::Global && callable->s == "collections OrderedDict") {
            push(mk(Value::Dict));
          } else {
            auto v = mk(Value::Reduce); v->items = {callable, args}; push(v);
          }
          break;
        }
        case 'b': pop(); break;                                   // BUILD: object state is dropped
        default:
          throw std::runtime_error("pickle: unsupported opcode " + std::to_string((int)op));
      }
    }
  }

 private:
  uint8_t u8() { return *take(1); }
  const uint8_t* take(size_t k) {
    if (pos_ + k > n_) throw std::runtime_error("pickle: truncated");
    const uint8_t* p = d_ + pos_;
    pos_ += k;
    return p;
  }
  std::string line() {
    std::string s;
    for (uint8_t c = u8(); c != '\n'; c = u8()) s.push_back((char)c);
    return s;
  }
  void str(size_t len) { auto v = mk(Value::Str); v->s.assign((const char*)take(len), len); push(v); }
  void push(ValuePtr v) { stack_.push_back(std::move(v)); }
  ValuePtr& top() {
    if (stack_.empty()) throw std::runtime_error("pickle: empty stack");
    return stack_.back();
  }
  ValuePtr pop() { ValuePtr v = top(); stack_.pop_back(); return v; }
  ValuePtr get(uint32_t k) {
    auto it = memo_.find(k);
    if (it == memo_.end()) throw std::runtime_error("pickle: memo miss");
    return it->second;
  }
  std::vector<ValuePtr> pop_to_mark() {
    std::vector<ValuePtr> xs;
    for (;;) {
      ValuePtr v = pop();
      if (v->kind == Value::Mark) break;
      xs.push_back(v);
    }
    return std::vector<ValuePtr>(xs.rbegin(), xs.rend());
  }
  const uint8_t* d_;
  size_t n_, pos_ = 0;
  std::vector<ValuePtr> stack_;
  std::map<uint32_t, ValuePtr> memo_;
};

inline const Value* dict_get(const Value* d, const std::string& key) {
  if (d->kind != Value::Dict) throw std::runtime_error("expected dict");
  for (auto& kv : d->dict)
    if (kv.first->kind == Value::Str && kv.first->s == key) return kv.second.get();
  return nullptr;
}

}  // namespace detail

// pickle.rs:186-267.  `dict_path` names the entry of the top-level dict that holds the state
// dict (None in the reference = the top level itself).
class PickledModel {
 public:
  static std::unique_ptr<PickledModel> load_file(const std::string& path, const char* dict_path = nullptr) {
    std::unique_ptr<PickledModel> m(new PickledModel(path));
    const auto files = detail::read_zip_directory(m->mapping.data(), m->mapping.size());
    auto pkl = files.find("data.pkl");
    if (pkl == files.end()) throw std::runtime_error("data.pkl not found");
    detail::Unpickler up(m->mapping.data() + pkl->second.data_start, pkl->second.size);
    const detail::ValuePtr root = up.load();
    const detail::Value* dict = root.get();
    if (dict_path) {
      dict = detail::dict_get(dict, dict_path);
      if (!dict) throw std::runtime_error("key not found");
    }
    if (dict->kind != detail::Value::Dict) throw std::runtime_error("expected dict");
    m->tensors_from_dict(dict, files);
    return m;
  }
  const PickledTensor& tensor(const std::string& name) const {
    auto it = tensors.find(name);
    if (it == tensors.end()) throw std::runtime_error("tensor " + name + " not found");
    return it->second;
  }
  // The bytes load_tensor (pickle.rs:322-338) copies to the device.
  const uint8_t* bytes(const PickledTensor& t) const { return mapping.data() + t.begin; }

  MappedBuffer mapping;
  std::map<std::string, PickledTensor> tensors;

 private:
  explicit PickledModel(const std::string& path) : mapping(path) {}

  // pickle.rs:130-184
  void tensors_from_dict(const detail::Value* dict, const std::map<std::string, ZipMember>& files) {
    using detail::Value;
    for (auto& kv : dict->dict) {
      if (kv.first->kind != Value::Str || kv.first->s == "_metadata") continue;
      const Value* v = kv.second.get();
      // torch._utils._rebuild_tensor_v2(storage, storage_offset, size, stride, requires_grad, hooks)
      if (v->kind != Value::Reduce || v->items[0]->kind != Value::Global ||
          v->items[0]->s != "torch._utils _rebuild_tensor_v2" || v->items[1]->kind != Value::Tuple ||
          v->items[1]->items.size() < 4)
        throw std::runtime_error("entry " + kv.first->s + " is not a tensor");
      const auto& a = v->items[1]->items;
      // persistent id ('storage', <storage class>, key, location, numel)
      if (a[0]->kind != Value::PersId || a[0]->items[0]->kind != Value::Tuple ||
          a[0]->items[0]->items.size() < 5)
        throw std::runtime_error("entry " + kv.first->s + ": unexpected storage record");
      const auto& st = a[0]->items[0]->items;
      if (st[1]->kind != Value::Global || st[2]->kind != Value::Str)
        throw std::runtime_error("entry " + kv.first->s + ": unexpected storage record");
      PickledTensor t;
      const std::string& cls = st[1]->s;
      if (cls == "torch FloatStorage") t.dtype = TensorDataType::F32;
      else if (cls == "torch HalfStorage") t.dtype = TensorDataType::F16;
      else if (cls == "torch LongStorage") t.dtype = TensorDataType::I64;
      else throw std::runtime_error("unsupported dtype: " + cls);
      const size_t el = element_size(t.dtype);
      auto f = files.find(st[2]->s);
      if (f == files.end()) throw std::runtime_error("tensor data not found: " + st[2]->s);
      t.begin = f->second.data_start;
      t.end = t.begin + f->second.size;
      if (a[1]->kind != Value::Int || a[2]->kind != Value::Tuple || a[3]->kind != Value::Tuple ||
          a[2]->items.size() != a[3]->items.size())
        throw std::runtime_error("entry " + kv.first->s + ": unexpected tensor record");
      const int64_t off = a[1]->i;
      if (off < 0 || (uint64_t)off > (t.end - t.begin) / el) throw std::runtime_error("invalid storage offset");
      t.begin += (size_t)off * el;
      size_t largest = 0;
      for (size_t k = 0; k < a[2]->items.size(); k++) {
        if (a[2]->items[k]->kind != Value::Int || a[3]->items[k]->kind != Value::Int ||
            a[2]->items[k]->i < 0 || a[3]->items[k]->i < 0)
          throw std::runtime_error("entry " + kv.first->s + ": unexpected tensor record");
        t.shape.push_back((size_t)a[2]->items[k]->i);
        t.stride.push_back((size_t)a[3]->items[k]->i);
        if (t.shape.back() == 0) throw std::runtime_error("entry " + kv.first->s + ": empty dimension");
        size_t reach;
        if (__builtin_mul_overflow(t.shape.back() - 1, t.stride.back(), &reach) ||
            __builtin_add_overflow(largest, reach, &largest))
          throw std::runtime_error("invalid tensor size");
      }
      if (!t.shape.empty()) {
        // trimmed to the addressed span (pickle.rs:160-168)
        size_t span;
        if (__builtin_add_overflow(largest, (size_t)1, &span) || __builtin_mul_overflow(span, el, &span) ||
            span > t.end - t.begin)
          throw std::runtime_error("invalid tensor size");
        t.end = t.begin + span;
      }
      tensors.emplace(kv.first->s, std::move(t));
    }
  }
};

// pickle.rs:269-320: a directory with pytorch_model.bin.index.json, whose "weight_map" object
// maps tensor names to shard file names; shards are opened in the order the map names them.
class ShardedModel {
 public:
  static std::unique_ptr<ShardedModel> load_huggingface(const std::string& dir) {
    std::unique_ptr<ShardedModel> m(new ShardedModel);
    MappedBuffer idx(dir + "/pytorch_model.bin.index.json");
    const std::string text((const char*)idx.data(), idx.size());
    std::map<std::string, size_t> shard_index;
    for (auto& kv : weight_map(text)) {
      auto it = shard_index.find(kv.second);
      if (it == shard_index.end()) {
        m->shards_.push_back(PickledModel::load_file(dir + "/" + kv.second));
        it = shard_index.emplace(kv.second, m->shards_.size() - 1).first;
      }
      m->index_[kv.first] = it->second;
    }
    return m;
  }
  // The shard and record load_tensor (pickle.rs:300-320) copies from.
  std::pair<const PickledModel*, const PickledTensor*> find(const std::string& name) const {
    auto it = index_.find(name);
    if (it == index_.end()) throw std::runtime_error("tensor " + name + " not found");
    const PickledModel* shard = shards_[it->second].get();
    return {shard, &shard->tensor(name)};
  }
  size_t shard_count() const { return shards_.size(); }

 private:
  // The string -> string members of the "weight_map" object, sorted by name like the
  // reference's BTreeMap.  A JSON reader for exactly this shape: strings with escapes, nesting
  // of other values skipped.
  static std::map<std::string, std::string> weight_map(const std::string& t) {
    size_t p = t.find("\"weight_map\"");
    if (p == std::string::npos) throw std::runtime_error("weight_map not found");
    p = t.find('{', p);
    if (p == std::string::npos) throw std::runtime_error("weight_map is not an object");
    std::map<std::string, std::string> out;
    auto ws = [&] { while (p < t.size() && (t[p] == ' ' || t[p] == '\n' || t[p] == '\r' || t[p] == '\t')) p++; };
    auto str = [&] {
      if (p >= t.size() || t[p] != '"') throw std::runtime_error("index json: string expected");
      std::string s;
      for (p++; p < t.size() && t[p] != '"'; p++) {
        if (t[p] == '\\' && p + 1 < t.size()) {
          p++;
          s.push_back(t[p] == 'n' ? '\n' : t[p] == 't' ? '\t' : t[p]);
        } else {
          s.push_back(t[p]);
        }
      }
      if (p >= t.size()) throw std::runtime_error("index json: unterminated string");
      p++;
      return s;
    };
    p++;
    for (;;) {
      ws();
      if (p < t.size() && t[p] == '}') break;
      const std::string k = str();
      ws();
      if (p >= t.size() || t[p] != ':') throw std::runtime_error("index json: ':' expected");
      p++;
      ws();
      out[k] = str();
      ws();
      if (p < t.size() && t[p] == ',') { p++; continue; }
      if (p < t.size() && t[p] == '}') break;
      throw std::runtime_error("index json: ',' or '}' expected");
    }
    return out;
  }
  std::vector<std::unique_ptr<PickledModel>> shards_;
  std::map<std::string, size_t> index_;
};

}  // namespace adrastea
