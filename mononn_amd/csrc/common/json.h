// Minimal JSON document model, parser and pretty printer.  Used for the tuning specification
// files (the reference prints its protobuf spec with whitespace, primitive fields always present
// and original field names: mononn_engine/helpers/protobuf.cc:32-46) and for the GEMM
// backend_config string carried by custom-call instructions (gemm_impl.cc:182-231).
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <utility>
#include <vector>

namespace mononn {

class Json {
 public:
  enum Type { kNull, kBool, kInt, kDouble, kString, kArray, kObject };
  Json() : type_(kNull) {}
  Json(bool b) : type_(kBool), b_(b) {}
  Json(int v) : type_(kInt), i_(v) {}
  Json(int64_t v) : type_(kInt), i_(v) {}
  Json(uint64_t v) : type_(kInt), i_(static_cast<int64_t>(v)) {}
  Json(double v) : type_(kDouble), d_(v) {}
  Json(const char* s) : type_(kString), s_(s) {}
  Json(const std::string& s) : type_(kString), s_(s) {}
  static Json array() { Json j; j.type_ = kArray; return j; }
  static Json object() { Json j; j.type_ = kObject; return j; }

  Type type() const { return type_; }
  bool is_null() const { return type_ == kNull; }
  bool is_object() const { return type_ == kObject; }
  bool is_array() const { return type_ == kArray; }
  bool is_string() const { return type_ == kString; }
  bool is_number() const { return type_ == kInt || type_ == kDouble; }

  // accessors throw Error(kSpecError) on a type mismatch
  bool as_bool() const;
  int64_t as_int() const;        // accepts an integer-valued string too ("12")
  double as_double() const;
  const std::string& as_string() const;

  // arrays
  void push_back(Json v);
  size_t size() const;
  const Json& at(size_t i) const;
  const std::vector<Json>& items() const { return arr_; }

  // objects (insertion ordered)
  Json& operator[](const std::string& key);         // inserts null when absent
  const Json* find(const std::string& key) const;   // nullptr when absent
  const Json& at(const std::string& key) const;     // throws when absent
  bool contains(const std::string& key) const { return find(key) != nullptr; }
  const std::vector<std::pair<std::string, Json>>& members() const { return obj_; }

  std::string dump(int indent = 1) const;
  static Json parse(const std::string& text);       // throws Error(kParseError)

 private:
  void dump_to(std::string& out, int indent, int depth) const;
  Type type_;
  bool b_ = false;
  int64_t i_ = 0;
  double d_ = 0;
  std::string s_;
  std::vector<Json> arr_;
  std::vector<std::pair<std::string, Json>> obj_;
};

}  // namespace mononn
