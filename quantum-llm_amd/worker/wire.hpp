// Text in, text out: the two ends of the worker's line protocol.
//
// A command is one line of tab-separated fields, a reply one line of JSON
// (runtime/tools/moe_vm_runner.cpp:655-1470 is the runner whose wire format
// this worker speaks).  FieldCursor walks the fields of a command with typed
// reads; JsonLine assembles a reply and writes it with one flush.
#pragma once

#include <charconv>
#include <cstdint>
#include <ostream>
#include <span>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

namespace qllm::wire {

struct ProtocolError final : std::runtime_error {
  using std::runtime_error::runtime_error;
};

[[noreturn]] inline void fail(std::string_view message) {
  throw ProtocolError(std::string(message));
}

inline void expect(bool holds, std::string_view message) {
  if (!holds) fail(message);
}

// Strict decimal: the whole text must be the number.
template <typename Integer>
[[nodiscard]] Integer decimal(std::string_view text) {
  Integer value{};
  const auto* last = text.data() + text.size();
  const auto parsed = std::from_chars(text.data(), last, value);
  expect(!text.empty() && parsed.ec == std::errc{} && parsed.ptr == last,
         "worker command holds a malformed number");
  return value;
}

class FieldCursor final {
 public:
  explicit FieldCursor(std::string_view line) {
    std::size_t start = 0U;
    while (true) {
      const auto tab = line.find('\t', start);
      if (tab == std::string_view::npos) {
        fields_.push_back(line.substr(start));
        break;
      }
      fields_.push_back(line.substr(start, tab - start));
      start = tab + 1U;
    }
  }
  [[nodiscard]] std::size_t total() const noexcept { return fields_.size(); }
  [[nodiscard]] std::size_t left() const noexcept { return fields_.size() - at_; }
  [[nodiscard]] bool done() const noexcept { return at_ == fields_.size(); }
  [[nodiscard]] std::string_view text() { return fields_.at(at_++); }
  [[nodiscard]] std::uint64_t natural() { return decimal<std::uint64_t>(text()); }
  [[nodiscard]] std::int64_t integer() { return decimal<std::int64_t>(text()); }
  // consumes the next field when it is `word`
  [[nodiscard]] bool keyword(std::string_view word) noexcept {
    if (done() || fields_[at_] != word) return false;
    ++at_;
    return true;
  }

 private:
  std::vector<std::string_view> fields_;
  std::size_t at_{};
};

// Comma-separated token ids, every one below `vocabulary`; the empty text is
// the empty list.
[[nodiscard]] inline std::vector<std::uint32_t> token_list(std::string_view text,
                                                           std::uint32_t vocabulary) {
  std::vector<std::uint32_t> tokens;
  for (std::size_t start = 0U; start < text.size();) {
    auto stop = text.find(',', start);
    if (stop == std::string_view::npos) stop = text.size();
    const auto token = decimal<std::uint64_t>(text.substr(start, stop - start));
    expect(token < vocabulary, "token is outside model vocabulary");
    tokens.push_back(static_cast<std::uint32_t>(token));
    start = stop + 1U;
  }
  return tokens;
}

class JsonLine final {
 public:
  explicit JsonLine(std::string_view type) {
    body_ = "{\"type\":\"";
    body_ += type;
    body_ += '"';
  }
  JsonLine& number(std::string_view key, std::uint64_t value) {
    open(key);
    body_ += std::to_string(value);
    return *this;
  }
  JsonLine& boolean(std::string_view key, bool value) {
    open(key);
    body_ += value ? "true" : "false";
    return *this;
  }
  JsonLine& string(std::string_view key, std::string_view value) {
    open(key);
    quoted(value);
    return *this;
  }
  JsonLine& strings(std::string_view key, std::span<const std::string> values) {
    open(key);
    body_ += '[';
    for (std::size_t index = 0U; index < values.size(); ++index) {
      if (index) body_ += ',';
      quoted(values[index]);
    }
    body_ += ']';
    return *this;
  }
  JsonLine& numbers(std::string_view key, std::span<const std::uint32_t> values) {
    open(key);
    list(values);
    return *this;
  }
  // an array of {"id":..,"tokens":[..]} objects
  JsonLine& begin_items(std::string_view key) {
    open(key);
    body_ += '[';
    first_item_ = true;
    return *this;
  }
  JsonLine& item(std::uint64_t id, std::span<const std::uint32_t> tokens) {
    if (!first_item_) body_ += ',';
    first_item_ = false;
    body_ += "{\"id\":" + std::to_string(id) + ",\"tokens\":";
    list(tokens);
    body_ += '}';
    return *this;
  }
  JsonLine& end_items() {
    body_ += ']';
    return *this;
  }
  void send(std::ostream& out) {
    body_ += "}\n";
    out << body_ << std::flush;
  }

 private:
  void open(std::string_view key) {
    body_ += ",\"";
    body_ += key;
    body_ += "\":";
  }
  void list(std::span<const std::uint32_t> values) {
    body_ += '[';
    for (std::size_t index = 0U; index < values.size(); ++index) {
      if (index) body_ += ',';
      body_ += std::to_string(values[index]);
    }
    body_ += ']';
  }
  // quotes and backslashes escaped, line breaks and tabs flattened to spaces:
  // a reply is always one line
  void quoted(std::string_view value) {
    body_ += '"';
    for (const char c : value) {
      if (c == '"' || c == '\\') body_ += '\\';
      body_ += (c == '\n' || c == '\r' || c == '\t') ? ' ' : c;
    }
    body_ += '"';
  }
  std::string body_;
  bool first_item_{true};
};

}  // namespace qllm::wire
