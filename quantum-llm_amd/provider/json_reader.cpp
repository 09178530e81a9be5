#include "json_reader.hpp"

#include <charconv>

namespace qllm::json {
namespace {

constexpr int kMaximumDepth = 128;

class Reader final {
 public:
  explicit Reader(std::string_view text) : text_(text) {}

  Value document() {
    Value value = any(0);
    blanks();
    if (at_ != text_.size()) fail("unexpected data after the document");
    return value;
  }

 private:
  [[noreturn]] void fail(const char* what) const {
    throw Error(std::string("JSON: ") + what + " at byte " + std::to_string(at_));
  }
  void blanks() {
    while (at_ < text_.size() &&
           (text_[at_] == ' ' || text_[at_] == '\t' || text_[at_] == '\n' ||
            text_[at_] == '\r'))
      ++at_;
  }
  bool take(char expected) {
    if (at_ < text_.size() && text_[at_] == expected) {
      ++at_;
      return true;
    }
    return false;
  }
  void word(std::string_view expected) {
    if (text_.substr(at_, expected.size()) != expected) fail("unknown literal");
    at_ += expected.size();
  }

  Value any(int depth) {
    if (depth > kMaximumDepth) fail("nesting is too deep");
    blanks();
    if (at_ >= text_.size()) fail("unexpected end");
    switch (text_[at_]) {
      case '{': return object(depth);
      case '[': return array(depth);
      case '"': return Value(Value::Storage(string()));
      case 't': word("true"); return Value(Value::Storage(true));
      case 'f': word("false"); return Value(Value::Storage(false));
      case 'n': word("null"); return Value(Value::Storage(nullptr));
      default: return number();
    }
  }

  Value object(int depth) {
    ++at_;
    Object members;
    blanks();
    if (take('}')) return Value(Value::Storage(std::move(members)));
    for (;;) {
      blanks();
      if (at_ >= text_.size() || text_[at_] != '"') fail("object key expected");
      std::string key = string();
      blanks();
      if (!take(':')) fail("':' expected");
      if (!members.emplace(std::move(key), any(depth + 1)).second)
        fail("duplicate object key");
      blanks();
      if (take('}')) return Value(Value::Storage(std::move(members)));
      if (!take(',')) fail("',' or '}' expected");
    }
  }

  Value array(int depth) {
    ++at_;
    Array items;
    blanks();
    if (take(']')) return Value(Value::Storage(std::move(items)));
    for (;;) {
      items.push_back(any(depth + 1));
      blanks();
      if (take(']')) return Value(Value::Storage(std::move(items)));
      if (!take(',')) fail("',' or ']' expected");
    }
  }

  unsigned hex4() {
    if (at_ + 4 > text_.size()) fail("short \\u escape");
    unsigned value = 0;
    for (int index = 0; index < 4; ++index) {
      const char c = text_[at_++];
      value <<= 4;
      if (c >= '0' && c <= '9') value |= static_cast<unsigned>(c - '0');
      else if (c >= 'a' && c <= 'f') value |= static_cast<unsigned>(c - 'a' + 10);
      else if (c >= 'A' && c <= 'F') value |= static_cast<unsigned>(c - 'A' + 10);
      else fail("bad \\u escape");
    }
    return value;
  }

  static void utf8(std::string& out, unsigned code) {
    if (code < 0x80U) {
      out.push_back(static_cast<char>(code));
    } else if (code < 0x800U) {
      out.push_back(static_cast<char>(0xc0U | (code >> 6)));
      out.push_back(static_cast<char>(0x80U | (code & 0x3fU)));
    } else if (code < 0x10000U) {
      out.push_back(static_cast<char>(0xe0U | (code >> 12)));
      out.push_back(static_cast<char>(0x80U | ((code >> 6) & 0x3fU)));
      out.push_back(static_cast<char>(0x80U | (code & 0x3fU)));
    } else {
      out.push_back(static_cast<char>(0xf0U | (code >> 18)));
      out.push_back(static_cast<char>(0x80U | ((code >> 12) & 0x3fU)));
      out.push_back(static_cast<char>(0x80U | ((code >> 6) & 0x3fU)));
      out.push_back(static_cast<char>(0x80U | (code & 0x3fU)));
    }
  }

  std::string string() {
    ++at_;  // opening quote
    std::string out;
    for (;;) {
      if (at_ >= text_.size()) fail("unterminated string");
      const char c = text_[at_++];
      if (c == '"') return out;
      if (static_cast<unsigned char>(c) < 0x20U) fail("control byte in string");
      if (c != '\\') {
        out.push_back(c);
        continue;
      }
      if (at_ >= text_.size()) fail("unterminated escape");
      switch (text_[at_++]) {
        case '"': out.push_back('"'); break;
        case '\\': out.push_back('\\'); break;
        case '/': out.push_back('/'); break;
        case 'b': out.push_back('\b'); break;
        case 'f': out.push_back('\f'); break;
        case 'n': out.push_back('\n'); break;
        case 'r': out.push_back('\r'); break;
        case 't': out.push_back('\t'); break;
        case 'u': {
          unsigned code = hex4();
          if (code >= 0xd800U && code <= 0xdbffU) {
            if (!(take('\\') && take('u'))) fail("lone surrogate");
            const unsigned low = hex4();
            if (low < 0xdc00U || low > 0xdfffU) fail("lone surrogate");
            code = 0x10000U + ((code - 0xd800U) << 10) + (low - 0xdc00U);
          } else if (code >= 0xdc00U && code <= 0xdfffU) {
            fail("lone surrogate");
          }
          utf8(out, code);
          break;
        }
        default: fail("unknown escape");
      }
    }
  }

  Value number() {
    const std::size_t start = at_;
    bool integral = true;
    take('-');
    if (at_ >= text_.size() || text_[at_] < '0' || text_[at_] > '9')
      fail("value expected");
    if (text_[at_] == '0') {
      ++at_;
    } else {
      while (at_ < text_.size() && text_[at_] >= '0' && text_[at_] <= '9') ++at_;
    }
    if (take('.')) {
      integral = false;
      if (at_ >= text_.size() || text_[at_] < '0' || text_[at_] > '9')
        fail("digits expected after '.'");
      while (at_ < text_.size() && text_[at_] >= '0' && text_[at_] <= '9') ++at_;
    }
    if (at_ < text_.size() && (text_[at_] == 'e' || text_[at_] == 'E')) {
      integral = false;
      ++at_;
      if (at_ < text_.size() && (text_[at_] == '+' || text_[at_] == '-')) ++at_;
      if (at_ >= text_.size() || text_[at_] < '0' || text_[at_] > '9')
        fail("digits expected in exponent");
      while (at_ < text_.size() && text_[at_] >= '0' && text_[at_] <= '9') ++at_;
    }
    const std::string_view token = text_.substr(start, at_ - start);
    if (integral) {
      const char* const end = token.data() + token.size();
      if (token.front() == '-') {
        std::int64_t value{};
        const auto [stop, error] = std::from_chars(token.data(), end, value);
        if (error == std::errc{} && stop == end)
          return Value(Value::Storage(value));
      } else {
        std::uint64_t value{};
        const auto [stop, error] = std::from_chars(token.data(), end, value);
        if (error == std::errc{} && stop == end)
          return Value(Value::Storage(value));
      }
      fail("integer is out of range");
    }
    return Value(Value::Storage(Value::Real{std::string(token)}));
  }

  std::string_view text_;
  std::size_t at_{};
};

[[noreturn]] void wrong_type(std::string_view where, const char* wanted) {
  throw Error(std::string(where) + " must be " + wanted);
}

}  // namespace

const Object& Value::object(std::string_view where) const {
  if (const auto* value = std::get_if<Object>(&data_)) return *value;
  wrong_type(where, "an object");
}

const Array& Value::array(std::string_view where) const {
  if (const auto* value = std::get_if<Array>(&data_)) return *value;
  wrong_type(where, "an array");
}

const std::string& Value::string(std::string_view where) const {
  if (const auto* value = std::get_if<std::string>(&data_)) return *value;
  wrong_type(where, "a string");
}

bool Value::boolean(std::string_view where) const {
  if (const auto* value = std::get_if<bool>(&data_)) return *value;
  wrong_type(where, "a boolean");
}

std::uint64_t Value::u64(std::string_view where) const {
  if (const auto* value = std::get_if<std::uint64_t>(&data_)) return *value;
  if (const auto* value = std::get_if<std::int64_t>(&data_); value && *value >= 0)
    return static_cast<std::uint64_t>(*value);
  wrong_type(where, "a non-negative integer");
}

Value parse(std::string_view text) { return Reader(text).document(); }

const Value& required(const Object& object, std::string_view key,
                      std::string_view where) {
  const auto found = object.find(key);
  if (found == object.end())
    throw Error(std::string(where) + " is missing required key '" +
                std::string(key) + "'");
  return found->second;
}

}  // namespace qllm::json
