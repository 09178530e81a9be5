// What a worker implementation advertises to the launcher
// (runtime/include/expert/runtime/worker_provider.hpp:12-21): a diagnostic
// name, a priority and the capability table it serves.
#pragma once

#include "expert/runtime/model_descriptor.hpp"

#include <cstdint>
#include <string>
#include <vector>

namespace expert::runtime {

using WorkerProviderEntry = int (*)(int argc, char** argv);

struct WorkerProviderDefinition final {
  std::string name;
  std::uint32_t priority{};
  std::vector<KernelCapability> capabilities;
  WorkerProviderEntry entry{};
};

}  // namespace expert::runtime
