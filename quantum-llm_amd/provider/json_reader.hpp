// A small JSON reader for the artifact manifest (RFC 8259 documents as the
// artifact compiler writes them).  Integers without fraction or exponent keep
// their exact value; objects reject duplicate keys; accessors throw
// json::Error naming the place, like expert::core::json of the reference
// (core/include/expert/core/json.hpp:16-56), whose manifest reader this serves.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <string_view>
#include <variant>
#include <vector>

namespace qllm::json {

class Error final : public std::runtime_error {
 public:
  using std::runtime_error::runtime_error;
};

class Value;
using Array = std::vector<Value>;
using Object = std::map<std::string, Value, std::less<>>;

class Value final {
 public:
  struct Real final {
    std::string token;  // the number as written
  };
  using Storage = std::variant<std::nullptr_t, bool, std::int64_t, std::uint64_t,
                               Real, std::string, Array, Object>;
  Value() : data_(nullptr) {}
  explicit Value(Storage data) : data_(std::move(data)) {}

  [[nodiscard]] const Object& object(std::string_view where) const;
  [[nodiscard]] const Array& array(std::string_view where) const;
  [[nodiscard]] const std::string& string(std::string_view where) const;
  [[nodiscard]] bool boolean(std::string_view where) const;
  [[nodiscard]] std::uint64_t u64(std::string_view where) const;

 private:
  Storage data_;
};

[[nodiscard]] Value parse(std::string_view text);
// object[key], or Error("<where> is missing required key '<key>'")
[[nodiscard]] const Value& required(const Object& object, std::string_view key,
                                    std::string_view where);

}  // namespace qllm::json
