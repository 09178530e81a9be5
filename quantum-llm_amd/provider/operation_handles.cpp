// The two result handles of the provider boundary
// (runtime/include/expert/runtime/program_executor.hpp:136-160, 214-238;
// defined in the reference by runtime/src/program_executor.cpp).  A handle
// wraps the provider's poll and cancel closures; once poll() has produced the
// result, or cancel() has been called, it stays terminal.
#include "expert/runtime/program_executor.hpp"

#include <exception>
#include <string>
#include <utility>

namespace expert::runtime {
namespace {

// What both handles share: the closures, and whether the result has been
// handed out or the work cancelled.  A poll that throws cancels the work and
// reports the failure as the result (program_executor.cpp:50-79).
template <typename Result>
struct HandleCore {
  std::function<std::optional<Result>()> poll;
  std::function<void()> cancel;
  bool terminal{};

  [[nodiscard]] bool live() const noexcept {
    return !terminal && static_cast<bool>(poll);
  }
  std::optional<Result> take(const char* who) {
    if (!live()) return std::nullopt;
    std::string failure;
    try {
      auto result = poll();
      if (result) terminal = true;
      return result;
    } catch (const std::exception& error) {
      failure = std::string(who) + " poll failed: " + error.what();
    } catch (...) {
      failure = std::string(who) + " poll failed";
    }
    stop();
    Result failed{};
    failed.status = {ErrorCode::internal, std::move(failure)};
    return failed;
  }
  void stop() noexcept {
    if (terminal) return;
    terminal = true;
    try {
      if (cancel) cancel();
    } catch (...) {
    }
  }
};

}  // namespace

struct OperationExecutionHandle::Core final
    : HandleCore<OperationExecutionResult> {};

OperationExecutionHandle::OperationExecutionHandle() = default;
OperationExecutionHandle::OperationExecutionHandle(
    OperationExecutionHandle&&) noexcept = default;
OperationExecutionHandle& OperationExecutionHandle::operator=(
    OperationExecutionHandle&& other) noexcept {
  if (this != &other) {
    cancel();
    core_ = std::move(other.core_);
  }
  return *this;
}
OperationExecutionHandle::~OperationExecutionHandle() { cancel(); }
OperationExecutionHandle::OperationExecutionHandle(
    std::unique_ptr<Core> core) noexcept
    : core_(std::move(core)) {}

bool OperationExecutionHandle::valid() const noexcept {
  return core_ && core_->live();
}
std::optional<OperationExecutionResult> OperationExecutionHandle::poll() {
  return core_ ? core_->take("operation provider") : std::nullopt;
}
void OperationExecutionHandle::cancel() noexcept {
  if (core_) core_->stop();
}
OperationExecutionHandle OperationExecutionHandle::from_callbacks(
    Poll poll, Cancel cancel) {
  if (!poll || !cancel) return {};
  auto core = std::make_unique<Core>();
  core->poll = std::move(poll);
  core->cancel = std::move(cancel);
  return OperationExecutionHandle(std::move(core));
}

struct ExactDecodeExecutionHandle::Core final
    : HandleCore<ExactDecodeExecutionResult> {};

ExactDecodeExecutionHandle::ExactDecodeExecutionHandle() = default;
ExactDecodeExecutionHandle::ExactDecodeExecutionHandle(
    ExactDecodeExecutionHandle&&) noexcept = default;
ExactDecodeExecutionHandle& ExactDecodeExecutionHandle::operator=(
    ExactDecodeExecutionHandle&& other) noexcept {
  if (this != &other) {
    cancel();
    core_ = std::move(other.core_);
  }
  return *this;
}
ExactDecodeExecutionHandle::~ExactDecodeExecutionHandle() { cancel(); }
ExactDecodeExecutionHandle::ExactDecodeExecutionHandle(
    std::unique_ptr<Core> core) noexcept
    : core_(std::move(core)) {}

bool ExactDecodeExecutionHandle::valid() const noexcept {
  return core_ && core_->live();
}
std::optional<ExactDecodeExecutionResult> ExactDecodeExecutionHandle::poll() {
  return core_ ? core_->take("exact decode provider") : std::nullopt;
}
void ExactDecodeExecutionHandle::cancel() noexcept {
  if (core_) core_->stop();
}
ExactDecodeExecutionHandle ExactDecodeExecutionHandle::from_callbacks(
    Poll poll, Cancel cancel) {
  if (!poll || !cancel) return {};
  auto core = std::make_unique<Core>();
  core->poll = std::move(poll);
  core->cancel = std::move(cancel);
  return ExactDecodeExecutionHandle(std::move(core));
}

}  // namespace expert::runtime
