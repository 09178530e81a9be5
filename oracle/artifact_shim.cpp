// C-callable shim over an artifact reader and provider registry that follow
// the declarations of namespace expert::runtime.  TEST INFRASTRUCTURE ONLY:
// it exists so that tests can print what a reader made of its input and compare
// two readers line by line.  Built twice by oracle/Makefile:
//   - with the reference sources runtime/src/{model_descriptor,
//     execution_provider,model_artifact,model_tensor_store,sha256,
//     expert_catalog,expert_record}.cpp and core/src/json.cpp, read where they
//     lie in the reference tree, into oracle/_ref/libqllm_ref_artifact.so
//     (functions qref_*);
//   - with -DQLLM_SHIM_OVER_PRODUCT against this repository's headers and
//     libqllm_provider.so, into oracle/libqllm_provider_probe.so (functions
//     qprobe_*).
// The shim adds no logic: it calls the reader's functions and prints their
// results with one writer (descriptor_dump.hpp, registry_probe.hpp).
#include "expert/runtime/model_artifact.hpp"
#include "expert/runtime/model_descriptor.hpp"
#include "expert/runtime/model_tensor_store.hpp"
#include "expert/runtime/sha256.hpp"

#include "descriptor_dump.hpp"
#include "registry_probe.hpp"

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <memory>
#include <string>

namespace er = expert::runtime;

#ifdef QLLM_SHIM_OVER_PRODUCT
#define SHIM(name) qprobe_##name
#else
#define SHIM(name) qref_##name
#endif

namespace {

void copy_text(const std::string& text, char* buffer, std::size_t capacity,
               std::size_t* bytes) {
  if (bytes) *bytes = text.size();
  if (buffer && capacity) {
    const std::size_t count = std::min(text.size(), capacity - 1U);
    std::memcpy(buffer, text.data(), count);
    buffer[count] = '\0';
  }
}

// status code; the message goes where the dump would have gone
int report(const er::Status& status, char* buffer, std::size_t capacity,
           std::size_t* bytes) {
  copy_text(std::string(status.message()), buffer, capacity, bytes);
  return static_cast<int>(status.code());
}

er::Sha256Digest digest_of(const std::uint8_t* bytes) {
  er::Sha256Digest digest{};
  if (bytes) std::memcpy(digest.data(), bytes, digest.size());
  return digest;
}

struct Artifact {
  er::ModelArtifact artifact;
  er::MappedModelTensorStore store;
};

}  // namespace

extern "C" {

void SHIM(sha256)(const void* data, std::size_t bytes, std::uint8_t* digest) {
  const auto result = er::sha256({static_cast<const std::byte*>(data), bytes});
  std::memcpy(digest, result.data(), result.size());
}

int SHIM(model_descriptor_parse)(const char* text, std::size_t text_bytes,
                                const std::uint8_t* content_sha256,
                                std::uint64_t namespace_base, char* dump,
                                std::size_t capacity, std::size_t* dump_bytes) {
  const auto parsed = er::parse_model_descriptor_artifact(
      {text, text_bytes}, digest_of(content_sha256), namespace_base);
  if (!parsed.status.ok()) return report(parsed.status, dump, capacity, dump_bytes);
  copy_text(qllm::dump::model_descriptor(parsed.descriptor), dump, capacity,
            dump_bytes);
  return 0;
}

int SHIM(model_descriptor_load)(const char* path, std::uint64_t expected_bytes,
                               const std::uint8_t* expected_sha256,
                               const std::uint8_t* content_sha256,
                               std::uint64_t namespace_base, char* dump,
                               std::size_t capacity, std::size_t* dump_bytes) {
  const auto parsed = er::load_model_descriptor_artifact(
      path, expected_bytes, digest_of(expected_sha256), digest_of(content_sha256),
      namespace_base);
  if (!parsed.status.ok()) return report(parsed.status, dump, capacity, dump_bytes);
  copy_text(qllm::dump::model_descriptor(parsed.descriptor), dump, capacity,
            dump_bytes);
  return 0;
}

// the reference's ExecutionProviderRegistry and compile_model_program
// (runtime/src/execution_provider.cpp, model_descriptor.cpp:374-490)
void SHIM(model_program_bind)(const char* text, std::size_t text_bytes,
                             const std::uint8_t* content_sha256,
                             std::uint64_t namespace_base, const char* providers,
                             int executable, char* dump, std::size_t capacity,
                             std::size_t* dump_bytes) {
  copy_text(qllm::dump::bind_report({text, text_bytes}, digest_of(content_sha256),
                                    namespace_base, providers, executable != 0),
            dump, capacity, dump_bytes);
}

int SHIM(artifact_open)(const char* root, std::uint32_t mtp_draft_depth,
                       int map_tensors, void** out, char* message,
                       std::size_t capacity) {
  *out = nullptr;
  auto handle = std::make_unique<Artifact>();
  auto status = er::ModelArtifact::load(root, handle->artifact);
  if (status.ok() && mtp_draft_depth)
    status = handle->artifact.configure_mtp_draft_depth(mtp_draft_depth);
  if (status.ok() && map_tensors)
    status = er::MappedModelTensorStore::create(handle->artifact, handle->store);
  if (!status.ok()) return report(status, message, capacity, nullptr);
  *out = handle.release();
  return 0;
}

void SHIM(artifact_close)(void* artifact) { delete static_cast<Artifact*>(artifact); }

void SHIM(artifact_dump)(const void* artifact, char* dump, std::size_t capacity,
                        std::size_t* dump_bytes) {
  copy_text(qllm::dump::model_artifact(static_cast<const Artifact*>(artifact)->artifact),
            dump, capacity, dump_bytes);
}

int SHIM(artifact_tensor)(void* artifact, const char* name, const void** record,
                         std::uint64_t* record_bytes, char* message,
                         std::size_t capacity) {
  const auto resolved = static_cast<Artifact*>(artifact)->store.resolve(name);
  if (!resolved.status.ok()) return report(resolved.status, message, capacity, nullptr);
  *record = resolved.tensor->value.data;
  *record_bytes = resolved.tensor->value.bytes;
  return 0;
}

}  // extern "C"
