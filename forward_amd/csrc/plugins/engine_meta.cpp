// Engine sidecar: typed reader / writer of "<engine file>.meta" (see engine_meta.h).
//
// The reference goes through a JSON library (nlohmann::json) whose behaviour fixes the format:
// reading `value.get<int>()` accepts any JSON number (a fraction is cut off) or boolean and fails
// on everything else, a missing key reads as null (which fails for the scalars and is an empty
// sequence for the two arrays); writing `std::setw(4) << json` emits the keys in alphabetical
// order, four spaces per level, one array element per line, `[]` for an empty array.  The parser
// below is a plain recursive-descent JSON reader (objects, arrays, strings with escapes,
// numbers, true / false / null) that keeps only what the sidecar's keys need.
#include "engine_meta.h"

#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <fstream>
#include <map>
#include <sstream>

#include "../status.h"

namespace fwdmi {
namespace {

struct Value {
  enum Type { kNull, kBool, kInt, kFloat, kString, kArray, kObject } type = kNull;
  bool b = false;
  long long i = 0;
  double f = 0.0;
  std::string s;
  std::vector<Value> items;
  std::map<std::string, Value> members;
};

class Parser {
 public:
  explicit Parser(const std::string& text) : p_(text.data()), end_(text.data() + text.size()) {}

  bool document(Value* out) {
    if (!value(out, 0)) return false;
    skip_space();
    return p_ == end_ || fail("text after the document");
  }
  const std::string& error() const { return error_; }

 private:
  static constexpr int kMaxDepth = 64;
  const char* p_;
  const char* end_;
  std::string error_;

  bool fail(const char* what) {
    if (error_.empty()) error_ = what;
    return false;
  }
  void skip_space() {
    while (p_ < end_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) ++p_;
  }
  bool literal(const char* word) {
    const char* q = p_;
    for (; *word; ++word, ++q)
      if (q >= end_ || *q != *word) return fail("unknown literal");
    p_ = q;
    return true;
  }
  static void put_utf8(unsigned cp, std::string* s) {
    if (cp < 0x80) {
      s->push_back((char)cp);
    } else if (cp < 0x800) {
      s->push_back((char)(0xC0 | (cp >> 6)));
      s->push_back((char)(0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
      s->push_back((char)(0xE0 | (cp >> 12)));
      s->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      s->push_back((char)(0x80 | (cp & 0x3F)));
    } else {
      s->push_back((char)(0xF0 | (cp >> 18)));
      s->push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
      s->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      s->push_back((char)(0x80 | (cp & 0x3F)));
    }
  }
  bool hex4(unsigned* cp) {
    if (end_ - p_ < 4) return fail("short \\u escape");
    unsigned v = 0;
    for (int k = 0; k < 4; ++k) {
      const char c = *p_++;
      v <<= 4;
      if (c >= '0' && c <= '9') v |= (unsigned)(c - '0');
      else if (c >= 'a' && c <= 'f') v |= (unsigned)(c - 'a' + 10);
      else if (c >= 'A' && c <= 'F') v |= (unsigned)(c - 'A' + 10);
      else return fail("bad \\u escape");
    }
    *cp = v;
    return true;
  }
  bool string(std::string* out) {
    if (p_ >= end_ || *p_ != '"') return fail("expected a string");
    ++p_;
    out->clear();
    while (true) {
      if (p_ >= end_) return fail("unterminated string");
      const unsigned char c = (unsigned char)*p_++;
      if (c == '"') return true;
      if (c < 0x20) return fail("control character in a string");
      if (c != '\\') {
        out->push_back((char)c);
        continue;
      }
      if (p_ >= end_) return fail("unterminated escape");
      const char e = *p_++;
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
          unsigned cp = 0;
          if (!hex4(&cp)) return false;
          if (cp >= 0xD800 && cp <= 0xDBFF) {  // a surrogate pair
            unsigned lo = 0;
            if (end_ - p_ < 2 || p_[0] != '\\' || p_[1] != 'u') return fail("lone surrogate");
            p_ += 2;
            if (!hex4(&lo)) return false;
            if (lo < 0xDC00 || lo > 0xDFFF) return fail("lone surrogate");
            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
          } else if (cp >= 0xDC00 && cp <= 0xDFFF) {
            return fail("lone surrogate");
          }
          put_utf8(cp, out);
          break;
        }
        default: return fail("unknown escape");
      }
    }
  }
  bool number(Value* out) {
    const char* start = p_;
    if (p_ < end_ && *p_ == '-') ++p_;
    if (p_ >= end_ || *p_ < '0' || *p_ > '9') return fail("bad number");
    if (*p_ == '0') {
      ++p_;
    } else {
      while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
    }
    bool integral = true;
    if (p_ < end_ && *p_ == '.') {
      integral = false;
      ++p_;
      if (p_ >= end_ || *p_ < '0' || *p_ > '9') return fail("bad number");
      while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
    }
    if (p_ < end_ && (*p_ == 'e' || *p_ == 'E')) {
      integral = false;
      ++p_;
      if (p_ < end_ && (*p_ == '+' || *p_ == '-')) ++p_;
      if (p_ >= end_ || *p_ < '0' || *p_ > '9') return fail("bad number");
      while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
    }
    const std::string text(start, p_);
    if (integral) {
      errno = 0;
      const long long v = std::strtoll(text.c_str(), nullptr, 10);
      if (errno == 0) {
        out->type = Value::kInt;
        out->i = v;
        return true;
      }
    }
    out->type = Value::kFloat;
    out->f = std::strtod(text.c_str(), nullptr);
    return true;
  }
  bool value(Value* out, int depth) {
    if (depth > kMaxDepth) return fail("nested too deeply");
    skip_space();
    if (p_ >= end_) return fail("unexpected end of text");
    switch (*p_) {
      case '{': {
        ++p_;
        out->type = Value::kObject;
        skip_space();
        if (p_ < end_ && *p_ == '}') {
          ++p_;
          return true;
        }
        while (true) {
          skip_space();
          std::string key;
          if (!string(&key)) return false;
          skip_space();
          if (p_ >= end_ || *p_ != ':') return fail("expected ':'");
          ++p_;
          Value v;
          if (!value(&v, depth + 1)) return false;
          out->members[key] = std::move(v);  // a repeated key keeps its last value, as the library does
          skip_space();
          if (p_ < end_ && *p_ == ',') {
            ++p_;
            continue;
          }
          if (p_ < end_ && *p_ == '}') {
            ++p_;
            return true;
          }
          return fail("expected ',' or '}'");
        }
      }
      case '[': {
        ++p_;
        out->type = Value::kArray;
        skip_space();
        if (p_ < end_ && *p_ == ']') {
          ++p_;
          return true;
        }
        while (true) {
          Value v;
          if (!value(&v, depth + 1)) return false;
          out->items.push_back(std::move(v));
          skip_space();
          if (p_ < end_ && *p_ == ',') {
            ++p_;
            continue;
          }
          if (p_ < end_ && *p_ == ']') {
            ++p_;
            return true;
          }
          return fail("expected ',' or ']'");
        }
      }
      case '"':
        out->type = Value::kString;
        return string(&out->s);
      case 't':
        out->type = Value::kBool;
        out->b = true;
        return literal("true");
      case 'f':
        out->type = Value::kBool;
        out->b = false;
        return literal("false");
      case 'n':
        out->type = Value::kNull;
        return literal("null");
      default:
        return number(out);
    }
  }
};

// value.get<int>(): numbers and booleans convert, everything else is a type error.  A number
// that no int holds is refused (the library would wrap it silently).
bool as_int(const Value& v, int* out) {
  switch (v.type) {
    case Value::kBool:
      *out = v.b ? 1 : 0;
      return true;
    case Value::kInt:
      if (v.i < INT32_MIN || v.i > INT32_MAX) return false;
      *out = (int)v.i;
      return true;
    case Value::kFloat:
      if (!(v.f > -2147483649.0 && v.f < 2147483648.0)) return false;  // also refuses NaN
      *out = (int)v.f;  // the fraction is cut off
      return true;
    default:
      return false;
  }
}

const Value* find(const Value& doc, const char* key) {
  const auto it = doc.members.find(key);
  return it == doc.members.end() ? nullptr : &it->second;
}

bool read_int(const Value& doc, const char* key, int* out, std::string* why) {
  const Value* v = find(doc, key);
  if (!v || v->type == Value::kNull) {
    *why = std::string("key '") + key + "' is missing";
    return false;
  }
  if (!as_int(*v, out)) {
    *why = std::string("key '") + key + "' is not an integer";
    return false;
  }
  return true;
}

bool read_ints(const Value& doc, const char* key, std::vector<int>* out, std::string* why) {
  out->clear();
  const Value* v = find(doc, key);
  if (!v || v->type == Value::kNull) return true;  // an absent array reads as empty
  if (v->type != Value::kArray) {
    *why = std::string("key '") + key + "' is not an array";
    return false;
  }
  for (const Value& item : v->items) {
    int x = 0;
    if (!as_int(item, &x)) {
      *why = std::string("key '") + key + "' holds an element that is not an integer";
      return false;
    }
    out->push_back(x);
  }
  return true;
}

void put_string(const std::string& s, std::string* out) {
  out->push_back('"');
  for (const unsigned char c : s) {
    switch (c) {
      case '"': *out += "\\\""; break;
      case '\\': *out += "\\\\"; break;
      case '\b': *out += "\\b"; break;
      case '\f': *out += "\\f"; break;
      case '\n': *out += "\\n"; break;
      case '\r': *out += "\\r"; break;
      case '\t': *out += "\\t"; break;
      default:
        if (c < 0x20 || c == 0x7F) {
          char buf[8];
          std::snprintf(buf, sizeof(buf), "\\u%04x", (unsigned)c);
          *out += buf;
        } else {
          out->push_back((char)c);  // UTF-8 goes through as it is
        }
    }
  }
  out->push_back('"');
}

template <typename Seq>
void put_ints(const Seq& v, std::string* out) {
  if (v.empty()) {
    *out += "[]";
    return;
  }
  *out += "[\n";
  size_t k = 0;
  for (const int x : v) {
    *out += "        " + std::to_string(x);
    *out += ++k < v.size() ? ",\n" : "\n";
  }
  *out += "    ]";
}

}  // namespace

bool EngineMetaData::ParseMetaData(const std::string& json_text) {
  Value doc;
  Parser parser(json_text);
  if (!parser.document(&doc)) {
    set_error(FWDMI_ERR_BAD_ARG, "engine meta data: not JSON (%s)", parser.error().c_str());
    return false;
  }
  if (doc.type != Value::kObject) {
    set_error(FWDMI_ERR_BAD_ARG, "engine meta data: the document is not an object");
    return false;
  }
  EngineMetaData m;
  std::string why;
  int mode = 0;
  std::vector<int> unused, outputs;
  const Value* path = find(doc, "torch_module_path");
  bool ok = read_int(doc, "infer_mode", &mode, &why) && read_int(doc, "opt_batch_size", &m.opt_batch_size_, &why) &&
            read_int(doc, "max_batch_size", &m.max_batch_size_, &why) &&
            read_ints(doc, "unused_input_indices", &unused, &why) && read_ints(doc, "output_indices", &outputs, &why);
  if (ok && (!path || path->type != Value::kString)) {
    why = path && path->type != Value::kNull ? "key 'torch_module_path' is not a string" : "key 'torch_module_path' is missing";
    ok = false;
  }
  if (!ok) {
    set_error(FWDMI_ERR_BAD_ARG, "engine meta data: %s", why.c_str());
    return false;
  }
  m.mode_ = static_cast<InferMode>(mode);
  m.unused_input_indices_.insert(unused.begin(), unused.end());
  m.output_pos_.swap(outputs);
  m.torch_module_path_ = path->s;
  *this = std::move(m);
  return true;
}

bool EngineMetaData::LoadMetaData(const std::string& meta_file) {
  std::ifstream f(meta_file, std::ios::binary);
  if (!f.is_open()) {
    set_error(FWDMI_ERR_BAD_ARG, "engine meta data: cannot open '%s'", meta_file.c_str());
    return false;
  }
  std::stringstream ss;
  ss << f.rdbuf();
  return ParseMetaData(ss.str());
}

std::string EngineMetaData::ToJson() const {
  std::string out = "{\n";
  out += "    \"infer_mode\": " + std::to_string(static_cast<int>(mode_)) + ",\n";
  out += "    \"max_batch_size\": " + std::to_string(max_batch_size_) + ",\n";
  out += "    \"opt_batch_size\": " + std::to_string(opt_batch_size_) + ",\n";
  out += "    \"output_indices\": ";
  put_ints(output_pos_, &out);
  out += ",\n    \"torch_module_path\": ";
  put_string(torch_module_path_, &out);
  out += ",\n    \"unused_input_indices\": ";
  put_ints(unused_input_indices_, &out);
  out += "\n}\n";
  return out;
}

bool EngineMetaData::SaveMetaData(const std::string& meta_file) const {
  std::ofstream f(meta_file, std::ios::binary | std::ios::trunc);
  if (!f.is_open()) {
    set_error(FWDMI_ERR_BAD_ARG, "engine meta data: cannot create '%s'", meta_file.c_str());
    return false;
  }
  f << ToJson();
  f.close();
  if (!f) {
    set_error(FWDMI_ERR_BAD_ARG, "engine meta data: write to '%s' failed", meta_file.c_str());
    return false;
  }
  return true;
}

}  // namespace fwdmi
