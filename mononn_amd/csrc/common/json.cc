#include "common/json.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>

#include "common/status.h"

namespace mononn {

bool Json::as_bool() const {
  if (type_ == kBool) return b_;
  if (type_ == kInt) return i_ != 0;
  MONONN_FAIL(kSpecError) << "JSON value is not a bool";
}
int64_t Json::as_int() const {
  if (type_ == kInt) return i_;
  if (type_ == kDouble && std::floor(d_) == d_) return static_cast<int64_t>(d_);
  if (type_ == kString) {
    char* end = nullptr;
    long long v = std::strtoll(s_.c_str(), &end, 10);
    if (end && *end == 0 && !s_.empty()) return v;
  }
  MONONN_FAIL(kSpecError) << "JSON value is not an integer";
}
double Json::as_double() const {
  if (type_ == kInt) return static_cast<double>(i_);
  if (type_ == kDouble) return d_;
  if (type_ == kString) {
    char* end = nullptr;
    double v = std::strtod(s_.c_str(), &end);
    if (end && *end == 0 && !s_.empty()) return v;
  }
  MONONN_FAIL(kSpecError) << "JSON value is not a number";
}
const std::string& Json::as_string() const {
  MONONN_CHECK(type_ == kString, kSpecError) << "JSON value is not a string";
  return s_;
}
void Json::push_back(Json v) {
  if (type_ == kNull) type_ = kArray;
  MONONN_CHECK(type_ == kArray, kSpecError) << "push_back on a non-array";
  arr_.push_back(std::move(v));
}
size_t Json::size() const { return type_ == kArray ? arr_.size() : obj_.size(); }
const Json& Json::at(size_t i) const {
  MONONN_CHECK(type_ == kArray && i < arr_.size(), kSpecError) << "array index out of range";
  return arr_[i];
}
Json& Json::operator[](const std::string& key) {
  if (type_ == kNull) type_ = kObject;
  MONONN_CHECK(type_ == kObject, kSpecError) << "member access on a non-object";
  for (auto& kv : obj_)
    if (kv.first == key) return kv.second;
  obj_.emplace_back(key, Json());
  return obj_.back().second;
}
const Json* Json::find(const std::string& key) const {
  if (type_ != kObject) return nullptr;
  for (auto& kv : obj_)
    if (kv.first == key) return &kv.second;
  return nullptr;
}
const Json& Json::at(const std::string& key) const {
  const Json* j = find(key);
  MONONN_CHECK(j != nullptr, kSpecError) << "missing key '" << key << "'";
  return *j;
}

static void escape_to(std::string& out, const std::string& s) {
  out.push_back('"');
  for (unsigned char c : s) {
    switch (c) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\t': out += "\\t"; break;
      case '\r': out += "\\r"; break;
      default:
        if (c < 0x20) {
          char buf[8];
          std::snprintf(buf, sizeof buf, "\\u%04x", c);
          out += buf;
        } else {
          out.push_back(static_cast<char>(c));
        }
    }
  }
  out.push_back('"');
}

void Json::dump_to(std::string& out, int indent, int depth) const {
  auto nl = [&](int d) {
    if (indent > 0) {
      out.push_back('\n');
      out.append(static_cast<size_t>(indent * d), ' ');
    }
  };
  switch (type_) {
    case kNull: out += "null"; break;
    case kBool: out += b_ ? "true" : "false"; break;
    case kInt: out += std::to_string(i_); break;
    case kDouble: {
      char buf[40];
      std::snprintf(buf, sizeof buf, "%.17g", d_);
      out += buf;
      break;
    }
    case kString: escape_to(out, s_); break;
    case kArray:
      if (arr_.empty()) { out += "[]"; break; }
      out.push_back('[');
      for (size_t i = 0; i < arr_.size(); ++i) {
        nl(depth + 1);
        arr_[i].dump_to(out, indent, depth + 1);
        if (i + 1 < arr_.size()) out.push_back(',');
      }
      nl(depth);
      out.push_back(']');
      break;
    case kObject:
      if (obj_.empty()) { out += "{}"; break; }
      out.push_back('{');
      for (size_t i = 0; i < obj_.size(); ++i) {
        nl(depth + 1);
        escape_to(out, obj_[i].first);
        out += indent > 0 ? ": " : ":";
        obj_[i].second.dump_to(out, indent, depth + 1);
        if (i + 1 < obj_.size()) out.push_back(',');
      }
      nl(depth);
      out.push_back('}');
      break;
  }
}
std::string Json::dump(int indent) const {
  std::string out;
  dump_to(out, indent, 0);
  return out;
}

namespace {
struct P {
  const std::string& s;
  size_t i = 0;
  void ws() { while (i < s.size() && (s[i] == ' ' || s[i] == '\n' || s[i] == '\t' || s[i] == '\r')) ++i; }
  [[noreturn]] void fail(const char* what) { MONONN_FAIL(kParseError) << "JSON: " << what << " at offset " << i; }
  Json value() {
    ws();
    if (i >= s.size()) fail("unexpected end");
    char c = s[i];
    if (c == '{') {
      ++i;
      Json o = Json::object();
      ws();
      if (i < s.size() && s[i] == '}') { ++i; return o; }
      while (true) {
        ws();
        if (i >= s.size() || s[i] != '"') fail("expected key string");
        std::string k = str();
        ws();
        if (i >= s.size() || s[i] != ':') fail("expected ':'");
        ++i;
        o[k] = value();
        ws();
        if (i < s.size() && s[i] == ',') { ++i; continue; }
        if (i < s.size() && s[i] == '}') { ++i; return o; }
        fail("expected ',' or '}'");
      }
    }
    if (c == '[') {
      ++i;
      Json a = Json::array();
      ws();
      if (i < s.size() && s[i] == ']') { ++i; return a; }
      while (true) {
        a.push_back(value());
        ws();
        if (i < s.size() && s[i] == ',') { ++i; continue; }
        if (i < s.size() && s[i] == ']') { ++i; return a; }
        fail("expected ',' or ']'");
      }
    }
    if (c == '"') return Json(str());
    if (s.compare(i, 4, "true") == 0) { i += 4; return Json(true); }
    if (s.compare(i, 5, "false") == 0) { i += 5; return Json(false); }
    if (s.compare(i, 4, "null") == 0) { i += 4; return Json(); }
    size_t st = i;
    bool is_double = false;
    if (i < s.size() && (s[i] == '-' || s[i] == '+')) ++i;
    while (i < s.size() && (isdigit(static_cast<unsigned char>(s[i])) || s[i] == '.' || s[i] == 'e' || s[i] == 'E' || s[i] == '-' || s[i] == '+')) {
      if (s[i] == '.' || s[i] == 'e' || s[i] == 'E') is_double = true;
      ++i;
    }
    if (st == i) fail("unexpected character");
    std::string num = s.substr(st, i - st);
    if (is_double) return Json(std::strtod(num.c_str(), nullptr));
    return Json(static_cast<int64_t>(std::strtoll(num.c_str(), nullptr, 10)));
  }
  std::string str() {
    ++i;
    std::string out;
    while (i < s.size() && s[i] != '"') {
      if (s[i] == '\\') {
        ++i;
        if (i >= s.size()) fail("bad escape");
        switch (s[i]) {
          case 'n': out.push_back('\n'); break;
          case 't': out.push_back('\t'); break;
          case 'r': out.push_back('\r'); break;
          case 'b': out.push_back('\b'); break;
          case 'f': out.push_back('\f'); break;
          case 'u': {
            if (i + 4 >= s.size()) fail("bad \\u escape");
            unsigned v = static_cast<unsigned>(std::strtoul(s.substr(i + 1, 4).c_str(), nullptr, 16));
            if (v < 0x80) out.push_back(static_cast<char>(v));
            else if (v < 0x800) { out.push_back(static_cast<char>(0xC0 | (v >> 6))); out.push_back(static_cast<char>(0x80 | (v & 0x3F))); }
            else { out.push_back(static_cast<char>(0xE0 | (v >> 12))); out.push_back(static_cast<char>(0x80 | ((v >> 6) & 0x3F))); out.push_back(static_cast<char>(0x80 | (v & 0x3F))); }
            i += 4;
            break;
          }
          default: out.push_back(s[i]);
        }
        ++i;
      } else {
        out.push_back(s[i++]);
      }
    }
    if (i >= s.size()) fail("unterminated string");
    ++i;
    return out;
  }
};
}  // namespace

Json Json::parse(const std::string& text) {
  P p{text};
  Json v = p.value();
  p.ws();
  if (p.i != text.size()) p.fail("trailing characters");
  return v;
}

}  // namespace mononn
