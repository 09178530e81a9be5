// Expert Pack v1 reader.  What is accepted and rejected, and the messages,
// follow runtime/src/model_artifact.cpp:75-367 and
// runtime/src/model_tensor_store.cpp:30-195 of the reference for dense-only
// artifacts.
#include "expert/runtime/model_artifact.hpp"
#include "expert/runtime/model_tensor_store.hpp"
#include "expert/runtime/sha256.hpp"

#include "dense_record.hpp"

#include "json_reader.hpp"

#include <algorithm>
#include <atomic>
#include <cerrno>
#include <cstring>
#include <fstream>
#include <limits>
#include <map>
#include <sstream>
#include <stdexcept>
#include <thread>

#include <fcntl.h>
#include <sys/mman.h>
#include <unistd.h>

namespace expert::runtime {
namespace {

namespace json = qllm::json;

std::string slurp(const std::filesystem::path& path) {
  std::ifstream input(path, std::ios::binary);
  if (!input) throw std::invalid_argument("cannot open artifact metadata");
  std::ostringstream text;
  text << input.rdbuf();
  if (input.bad()) throw std::invalid_argument("cannot read artifact metadata");
  return text.str();
}

unsigned hex_digit(char c) {
  if (c >= '0' && c <= '9') return static_cast<unsigned>(c - '0');
  if (c >= 'a' && c <= 'f') return static_cast<unsigned>(c - 'a') + 10U;
  if (c >= 'A' && c <= 'F') return static_cast<unsigned>(c - 'A') + 10U;
  throw std::invalid_argument("artifact SHA-256 contains an invalid digit");
}

Sha256Digest digest_from_hex(std::string_view text) {
  if (text.size() != 64U)
    throw std::invalid_argument("artifact SHA-256 has the wrong length");
  Sha256Digest digest{};
  for (std::size_t index = 0; index < digest.size(); ++index)
    digest[index] = static_cast<std::byte>((hex_digit(text[2U * index]) << 4U) |
                                           hex_digit(text[2U * index + 1U]));
  return digest;
}

std::uint32_t narrow(std::uint64_t value, std::string_view what) {
  if (value > std::numeric_limits<std::uint32_t>::max())
    throw std::invalid_argument(std::string(what) + " exceeds uint32");
  return static_cast<std::uint32_t>(value);
}

// A manifest path must stay inside the artifact directory.
std::filesystem::path child_of(const std::filesystem::path& root,
                               std::string_view text) {
  const std::filesystem::path relative(text);
  if (relative.empty() || relative.is_absolute() || relative.has_root_name() ||
      relative.has_root_directory())
    throw std::invalid_argument("artifact path is not relative");
  for (const auto& part : relative)
    if (part == "..") throw std::invalid_argument("artifact path escapes root");
  return root / relative;
}

const json::Value& member(const json::Object& object, std::string_view key,
                          std::string_view where) {
  return json::required(object, key, where);
}

bool known_encoding(const std::string& encoding) {
  static constexpr std::string_view kKnown[] = {"I8",   "F32",      "I64",
                                                "BF16", "FP4_E2M1", "MXFP6_E3M2"};
  return std::find(std::begin(kKnown), std::end(kKnown), encoding) !=
         std::end(kKnown);
}

ArtifactPack read_pack(const std::filesystem::path& root,
                       const json::Object& item) {
  ArtifactPack pack;
  pack.name = member(item, "name", "pack").string("pack.name");
  pack.kind = member(item, "kind", "pack").string("pack.kind");
  pack.path = child_of(root, pack.name);
  pack.bytes = member(item, "bytes", "pack").u64("pack.bytes");
  pack.sha256 = digest_from_hex(member(item, "sha256", "pack").string("pack.sha256"));
  return pack;
}

ArtifactDenseTensor read_tensor(const json::Object& item) {
  ArtifactDenseTensor tensor;
  tensor.name = member(item, "name", "tensor").string("tensor.name");
  tensor.pack = member(item, "pack", "tensor").string("tensor.pack");
  tensor.record_offset = member(item, "offset", "tensor").u64("tensor.offset");
  tensor.stored_bytes =
      member(item, "stored_bytes", "tensor").u64("tensor.stored_bytes");
  tensor.encoding =
      member(item, "stored_dtype", "tensor").string("tensor.stored_dtype");
  tensor.quant_abi = narrow(
      member(item, "quant_abi", "tensor").u64("tensor.quant_abi"), "tensor quant ABI");
  for (const auto& dimension :
       member(item, "source_shape", "tensor").array("tensor.shape"))
    tensor.shape.push_back(
        narrow(dimension.u64("tensor.dimension"), "tensor dimension"));
  const auto& sections =
      member(item, "sections", "tensor").object("tensor.sections");
  const auto& data = member(sections, "data", "sections").object("tensor.data");
  const auto& scales =
      member(sections, "scales", "sections").object("tensor.scales");
  tensor.data_offset = member(data, "offset", "data").u64("data.offset");
  tensor.data_bytes = member(data, "bytes", "data").u64("data.bytes");
  tensor.scale_offset = member(scales, "offset", "scales").u64("scales.offset");
  tensor.scale_bytes = member(scales, "bytes", "scales").u64("scales.bytes");
  tensor.payload_sha256 = digest_from_hex(
      member(item, "payload_sha256", "tensor").string("tensor.payload_sha256"));
  return tensor;
}

class MappedPack final {
 public:
  MappedPack() = default;
  MappedPack(const MappedPack&) = delete;
  MappedPack& operator=(const MappedPack&) = delete;
  ~MappedPack() {
    if (data_) ::munmap(const_cast<std::byte*>(data_), bytes_);
  }

  static Status open(const ArtifactPack& pack, std::shared_ptr<MappedPack>& out) {
    if (pack.bytes == 0U || pack.bytes > std::numeric_limits<std::size_t>::max())
      return {ErrorCode::invalid_argument,
              "dense artifact pack exceeds the address space"};
    auto mapped = std::make_shared<MappedPack>();
    mapped->bytes_ = static_cast<std::size_t>(pack.bytes);
    const int file = ::open(pack.path.c_str(), O_RDONLY);
    if (file < 0)
      return {ErrorCode::open_failed,
              std::string("cannot open dense artifact pack: ") +
                  std::strerror(errno)};
    void* const address =
        ::mmap(nullptr, mapped->bytes_, PROT_READ, MAP_PRIVATE, file, 0);
    const int map_error = errno;
    (void)::close(file);
    if (address == MAP_FAILED)
      return {ErrorCode::open_failed,
              std::string("cannot map dense artifact pack: ") +
                  std::strerror(map_error)};
    mapped->data_ = static_cast<const std::byte*>(address);
    if (!constant_time_equal(sha256({mapped->data_, mapped->bytes_}), pack.sha256))
      return {ErrorCode::checksum_mismatch,
              "dense artifact pack checksum mismatch"};
    out = std::move(mapped);
    return Status::success();
  }

  [[nodiscard]] const std::byte* data() const noexcept { return data_; }
  [[nodiscard]] std::size_t bytes() const noexcept { return bytes_; }

 private:
  const std::byte* data_{};
  std::size_t bytes_{};
};

}  // namespace

Status ModelArtifact::configure_mtp_draft_depth(std::uint32_t depth) noexcept {
  try {
    if (!model_.exact_decode_program || depth == 0U ||
        depth >= model_.max_context_tokens ||
        depth == std::numeric_limits<std::uint32_t>::max())
      throw std::invalid_argument("artifact cannot apply the requested MTP depth");
    ModelDescriptor candidate = model_;
    auto& decode = *candidate.exact_decode_program;
    const auto declared = decode.parameters.find("draft_depth");
    if (decode.abi_version < 2U || declared == decode.parameters.end() ||
        declared->second == 0U ||
        declared->second >= std::numeric_limits<std::uint32_t>::max() ||
        decode.maximum_emitted_tokens != declared->second + 1U)
      throw std::invalid_argument(
          "artifact does not declare an adjustable MTP policy");
    declared->second = depth;
    decode.maximum_emitted_tokens = depth + 1U;
    if (auto status = validate_model_descriptor(candidate); !status.ok())
      return status;
    model_ = std::move(candidate);
    return Status::success();
  } catch (const std::exception& error) {
    return {ErrorCode::invalid_argument, error.what()};
  }
}

Status ModelArtifact::load(const std::filesystem::path& root,
                           ModelArtifact& destination) noexcept {
  try {
    if (!destination.root_.empty() || !std::filesystem::is_directory(root) ||
        !std::filesystem::is_regular_file(root / "manifest.json"))
      return {ErrorCode::invalid_argument,
              "artifact destination is non-empty or manifest is absent"};
    const auto document = json::parse(slurp(root / "manifest.json"));
    const auto& format =
        member(document.object("manifest"), "format", "manifest")
            .object("manifest.format");
    const auto& name = member(format, "name", "format").string("format.name");
    const auto version = member(format, "version", "format").u64("format.version");
    if (name == "expert-pack" && version == 1U)
      return load_expert_pack_v1(root, destination);
    return {ErrorCode::invalid_argument,
            "no artifact storage adapter implements manifest format"};
  } catch (const std::exception& error) {
    return {ErrorCode::invalid_argument,
            std::string("invalid artifact manifest: ") + error.what()};
  }
}

const ArtifactPack* ModelArtifact::find_pack(std::string_view name) const noexcept {
  const auto found = std::find_if(
      packs_.begin(), packs_.end(),
      [name](const ArtifactPack& pack) { return pack.name == name; });
  return found == packs_.end() ? nullptr : &*found;
}

Status ModelArtifact::load_expert_pack_v1(const std::filesystem::path& root,
                                          ModelArtifact& destination) noexcept {
  try {
    if (!destination.root_.empty() || !std::filesystem::is_directory(root) ||
        !std::filesystem::is_regular_file(root / "manifest.json") ||
        !std::filesystem::is_regular_file(root / "COMPLETED"))
      return {ErrorCode::invalid_argument,
              "artifact destination is non-empty or container is incomplete"};
    const auto document = json::parse(slurp(root / "manifest.json"));
    const auto& manifest = document.object("manifest");
    const auto& format =
        member(manifest, "format", "manifest").object("manifest.format");
    if (member(format, "name", "format").string("format.name") != "expert-pack" ||
        member(format, "version", "format").u64("format.version") != 1U)
      return {ErrorCode::invalid_argument, "artifact is not Expert Pack v1"};
    const auto& integrity =
        member(manifest, "integrity", "manifest").object("manifest.integrity");
    const auto content_hash =
        digest_from_hex(member(integrity, "content_sha256", "integrity")
                            .string("integrity.content_sha256"));

    const auto& program =
        member(manifest, "model_program", "manifest").object("manifest.model_program");
    if (member(program, "format", "model_program").string("model_program.format") !=
        "expert-runtime-model-v1")
      return {ErrorCode::invalid_argument,
              "artifact model program format is unsupported"};
    const auto program_path = child_of(
        root, member(program, "path", "model_program").string("model_program.path"));
    auto parsed = load_model_descriptor_artifact(
        program_path,
        member(program, "bytes", "model_program").u64("model_program.bytes"),
        digest_from_hex(
            member(program, "sha256", "model_program").string("model_program.sha256")),
        content_hash, namespace_id_from_content_hash(content_hash));
    if (!parsed.status.ok()) return parsed.status;
    if (!parsed.descriptor.routed_components.empty())
      return {ErrorCode::invalid_argument,
              "artifact declares routed expert components, which this dense "
              "provider does not execute"};

    ModelArtifact candidate;
    candidate.root_ = root;
    candidate.model_ = std::move(parsed.descriptor);
    std::map<std::string, std::uint64_t, std::less<>> pack_bytes;
    for (const auto& value :
         member(manifest, "packs", "manifest").array("manifest.packs")) {
      ArtifactPack pack = read_pack(root, value.object("pack"));
      if ((pack.kind != "dense" && pack.kind != "experts") ||
          !std::filesystem::is_regular_file(pack.path) ||
          std::filesystem::file_size(pack.path) != pack.bytes ||
          !pack_bytes.emplace(pack.name, pack.bytes).second)
        throw std::invalid_argument("artifact pack index is invalid");
      candidate.packs_.push_back(std::move(pack));
    }
    for (const auto& value :
         member(manifest, "tensors", "manifest").array("manifest.tensors")) {
      ArtifactDenseTensor tensor = read_tensor(value.object("tensor"));
      const auto pack = pack_bytes.find(tensor.pack);
      if (pack == pack_bytes.end() || tensor.shape.empty() ||
          tensor.record_offset > pack->second ||
          tensor.stored_bytes > pack->second - tensor.record_offset ||
          !known_encoding(tensor.encoding))
        throw std::invalid_argument("dense tensor index is invalid");
      candidate.dense_tensors_.push_back(std::move(tensor));
    }
    if (!member(manifest, "experts", "manifest").array("manifest.experts").empty())
      throw std::invalid_argument(
          "dense-only artifact contains routed expert records");
    destination = std::move(candidate);
    return Status::success();
  } catch (const std::exception& error) {
    return {ErrorCode::invalid_argument,
            std::string("invalid model artifact: ") + error.what()};
  }
}

// ---- mapped tensor store ------------------------------------------------------

struct MappedModelTensorStore::Core final {
  std::map<std::string, std::shared_ptr<MappedPack>, std::less<>> packs;
  std::map<std::string, std::shared_ptr<const ImmutableModelTensor>, std::less<>>
      tensors;
};

MappedModelTensorStore::MappedModelTensorStore() = default;
MappedModelTensorStore::MappedModelTensorStore(MappedModelTensorStore&&) noexcept =
    default;
MappedModelTensorStore& MappedModelTensorStore::operator=(
    MappedModelTensorStore&&) noexcept = default;
MappedModelTensorStore::~MappedModelTensorStore() = default;

bool MappedModelTensorStore::valid() const noexcept { return core_ != nullptr; }

Status MappedModelTensorStore::create(const ModelArtifact& artifact,
                                      MappedModelTensorStore& destination) noexcept {
  try {
    if (destination.valid())
      return {ErrorCode::invalid_argument,
              "mapped tensor store destination is already initialized"};
    auto core = std::make_shared<Core>();
    // Packs are mapped and hashed side by side (a checksum is sequential
    // within a file, not across files); the first failure in index order is
    // the one reported.
    std::vector<const ArtifactPack*> dense;
    for (const auto& pack : artifact.packs())
      if (pack.kind == "dense") dense.push_back(&pack);
    std::vector<std::shared_ptr<MappedPack>> mapped(dense.size());
    std::vector<Status> opened(dense.size());
    {
      constexpr std::size_t kMaximumThreads = 8;
      std::atomic<std::size_t> next{0};
      const auto work = [&]() {
        for (std::size_t index = next++; index < dense.size(); index = next++) {
          try {
            opened[index] = MappedPack::open(*dense[index], mapped[index]);
          } catch (const std::exception& error) {
            opened[index] = {ErrorCode::internal, error.what()};
          }
        }
      };
      std::vector<std::thread> threads;
      for (std::size_t index = 1;
           index < std::min(dense.size(), kMaximumThreads); ++index)
        threads.emplace_back(work);
      work();
      for (auto& thread : threads) thread.join();
    }
    for (std::size_t index = 0; index < dense.size(); ++index) {
      if (!opened[index].ok()) return opened[index];
      if (!core->packs.emplace(dense[index]->name, std::move(mapped[index])).second)
        return {ErrorCode::invalid_argument,
                "dense artifact pack name is duplicated"};
    }
    for (const auto& entry : artifact.dense_tensors()) {
      const auto pack = core->packs.find(entry.pack);
      if (pack == core->packs.end() || entry.stored_bytes == 0U ||
          entry.record_offset > pack->second->bytes() ||
          entry.stored_bytes > pack->second->bytes() - entry.record_offset ||
          entry.data_offset > entry.stored_bytes ||
          entry.data_bytes > entry.stored_bytes - entry.data_offset ||
          entry.scale_offset > entry.stored_bytes ||
          entry.scale_bytes > entry.stored_bytes - entry.scale_offset)
        return {ErrorCode::invalid_argument,
                "dense tensor record is outside its mapped pack"};
      auto tensor = std::make_shared<ImmutableModelTensor>();
      tensor->name = entry.name;
      tensor->encoding = entry.encoding;
      tensor->quant_abi = entry.quant_abi;
      tensor->shape = entry.shape;
      tensor->data_offset = entry.data_offset;
      tensor->data_bytes = entry.data_bytes;
      tensor->scale_offset = entry.scale_offset;
      tensor->scale_bytes = entry.scale_bytes;
      tensor->value = {"artifact.dense-record.v1", "host.mmap.readonly",
                       pack->second, pack->second->data() + entry.record_offset,
                       entry.stored_bytes};
      if (!core->tensors.emplace(entry.name, std::move(tensor)).second)
        return {ErrorCode::invalid_argument,
                "dense artifact tensor name is duplicated"};
    }
    destination.core_ = std::move(core);
    return Status::success();
  } catch (const std::exception& error) {
    return {ErrorCode::internal,
            std::string("mapped model tensor store failed: ") + error.what()};
  }
}

ResolveModelTensorResult MappedModelTensorStore::resolve(std::string_view name) {
  if (!core_)
    return {{ErrorCode::invalid_argument,
             "mapped model tensor store is not initialized"},
            {}};
  const auto found = core_->tensors.find(name);
  if (found == core_->tensors.end())
    return {{ErrorCode::invalid_argument,
             "artifact tensor is absent from the dense index"},
            {}};
  return {Status::success(), found->second};
}

}  // namespace expert::runtime
