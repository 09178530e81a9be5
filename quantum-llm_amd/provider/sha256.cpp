#include "expert/runtime/sha256.hpp"

#include <algorithm>
#include <bit>
#include <cstring>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

namespace expert::runtime {
namespace {

// First 32 bits of the fractional parts of the cube roots of the first 64
// primes (FIPS 180-4, 4.2.2).
constexpr std::uint32_t kRound[64] = {
    0x428a2f98U, 0x71374491U, 0xb5c0fbcfU, 0xe9b5dba5U, 0x3956c25bU, 0x59f111f1U,
    0x923f82a4U, 0xab1c5ed5U, 0xd807aa98U, 0x12835b01U, 0x243185beU, 0x550c7dc3U,
    0x72be5d74U, 0x80deb1feU, 0x9bdc06a7U, 0xc19bf174U, 0xe49b69c1U, 0xefbe4786U,
    0x0fc19dc6U, 0x240ca1ccU, 0x2de92c6fU, 0x4a7484aaU, 0x5cb0a9dcU, 0x76f988daU,
    0x983e5152U, 0xa831c66dU, 0xb00327c8U, 0xbf597fc7U, 0xc6e00bf3U, 0xd5a79147U,
    0x06ca6351U, 0x14292967U, 0x27b70a85U, 0x2e1b2138U, 0x4d2c6dfcU, 0x53380d13U,
    0x650a7354U, 0x766a0abbU, 0x81c2c92eU, 0x92722c85U, 0xa2bfe8a1U, 0xa81a664bU,
    0xc24b8b70U, 0xc76c51a3U, 0xd192e819U, 0xd6990624U, 0xf40e3585U, 0x106aa070U,
    0x19a4c116U, 0x1e376c08U, 0x2748774cU, 0x34b0bcb5U, 0x391c0cb3U, 0x4ed8aa4aU,
    0x5b9cca4fU, 0x682e6ff3U, 0x748f82eeU, 0x78a5636fU, 0x84c87814U, 0x8cc70208U,
    0x90befffaU, 0xa4506cebU, 0xbef9a3f7U, 0xc67178f2U};

constexpr std::uint32_t kInitial[8] = {0x6a09e667U, 0xbb67ae85U, 0x3c6ef372U,
                                       0xa54ff53aU, 0x510e527fU, 0x9b05688cU,
                                       0x1f83d9abU, 0x5be0cd19U};

#if defined(__x86_64__)
// One or more 64-byte blocks with the x86 SHA extensions: the state lives in
// two registers as (A,B,E,F) and (C,D,G,H), each sha256rnds2 does two rounds,
// sha256msg1/msg2 extend the message schedule four words at a time.
__attribute__((target("sha,sse4.1,ssse3"))) void blocks_sha_ni(
    std::uint32_t state[8], const std::byte* data, std::size_t blocks) noexcept {
  const __m128i byte_swap =
      _mm_set_epi64x(0x0c0d0e0f08090a0bLL, 0x0405060700010203LL);
  __m128i low = _mm_loadu_si128(reinterpret_cast<const __m128i*>(state));       // DCBA
  __m128i high = _mm_loadu_si128(reinterpret_cast<const __m128i*>(state + 4));  // HGFE
  low = _mm_shuffle_epi32(low, 0xb1);                 // CDAB
  high = _mm_shuffle_epi32(high, 0x1b);               // EFGH
  __m128i abef = _mm_alignr_epi8(low, high, 8);       // ABEF
  __m128i cdgh = _mm_blend_epi16(high, low, 0xf0);    // CDGH
  const auto* constants = reinterpret_cast<const __m128i*>(kRound);
  for (; blocks; --blocks, data += 64) {
    const __m128i saved_abef = abef;
    const __m128i saved_cdgh = cdgh;
    __m128i words[4];
    for (int index = 0; index < 4; ++index)
      words[index] = _mm_shuffle_epi8(
          _mm_loadu_si128(reinterpret_cast<const __m128i*>(data) + index),
          byte_swap);
    for (int quad = 0; quad < 16; ++quad) {
      __m128i& current = words[quad & 3];
      if (quad >= 4) {
        // W[t..t+3] from W[t-16..], W[t-15..] (msg1), W[t-7..] and W[t-2..] (msg2)
        __m128i extended = _mm_sha256msg1_epu32(current, words[(quad + 1) & 3]);
        extended = _mm_add_epi32(
            extended,
            _mm_alignr_epi8(words[(quad + 3) & 3], words[(quad + 2) & 3], 4));
        current = _mm_sha256msg2_epu32(extended, words[(quad + 3) & 3]);
      }
      __m128i rounds = _mm_add_epi32(current, _mm_loadu_si128(constants + quad));
      cdgh = _mm_sha256rnds2_epu32(cdgh, abef, rounds);
      rounds = _mm_shuffle_epi32(rounds, 0x0e);
      abef = _mm_sha256rnds2_epu32(abef, cdgh, rounds);
    }
    abef = _mm_add_epi32(abef, saved_abef);
    cdgh = _mm_add_epi32(cdgh, saved_cdgh);
  }
  low = _mm_shuffle_epi32(abef, 0x1b);                // FEBA
  high = _mm_shuffle_epi32(cdgh, 0xb1);               // DCHG
  _mm_storeu_si128(reinterpret_cast<__m128i*>(state),
                   _mm_blend_epi16(low, high, 0xf0));          // DCBA
  _mm_storeu_si128(reinterpret_cast<__m128i*>(state + 4),
                   _mm_alignr_epi8(high, low, 8));             // HGFE
}

bool has_sha_extensions() noexcept {
  static const bool available = __builtin_cpu_supports("sha") &&
                                __builtin_cpu_supports("sse4.1") &&
                                __builtin_cpu_supports("ssse3");
  return available;
}
#endif

}  // namespace

Sha256Stream::Sha256Stream(bool portable) noexcept {
  std::copy(std::begin(kInitial), std::end(kInitial), h_);
#if defined(__x86_64__)
  accelerated_ = !portable && has_sha_extensions();
#else
  (void)portable;
#endif
}

void Sha256Stream::block(const std::byte* sixty_four_bytes) noexcept {
#if defined(__x86_64__)
  if (accelerated_) {
    blocks_sha_ni(h_, sixty_four_bytes, 1);
    return;
  }
#endif
  std::uint32_t schedule[64];
  for (int word = 0; word < 16; ++word) {
    const auto* bytes = reinterpret_cast<const unsigned char*>(sixty_four_bytes) + 4 * word;
    schedule[word] = (std::uint32_t{bytes[0]} << 24) |
                     (std::uint32_t{bytes[1]} << 16) |
                     (std::uint32_t{bytes[2]} << 8) | std::uint32_t{bytes[3]};
  }
  for (int word = 16; word < 64; ++word) {
    const std::uint32_t x = schedule[word - 15];
    const std::uint32_t y = schedule[word - 2];
    const std::uint32_t small0 = std::rotr(x, 7) ^ std::rotr(x, 18) ^ (x >> 3);
    const std::uint32_t small1 = std::rotr(y, 17) ^ std::rotr(y, 19) ^ (y >> 10);
    schedule[word] = schedule[word - 16] + small0 + schedule[word - 7] + small1;
  }
  std::uint32_t a = h_[0], b = h_[1], c = h_[2], d = h_[3];
  std::uint32_t e = h_[4], f = h_[5], g = h_[6], h = h_[7];
  for (int round = 0; round < 64; ++round) {
    const std::uint32_t big1 = std::rotr(e, 6) ^ std::rotr(e, 11) ^ std::rotr(e, 25);
    const std::uint32_t choose = (e & f) ^ (~e & g);
    const std::uint32_t first = h + big1 + choose + kRound[round] + schedule[round];
    const std::uint32_t big0 = std::rotr(a, 2) ^ std::rotr(a, 13) ^ std::rotr(a, 22);
    const std::uint32_t majority = (a & b) ^ (a & c) ^ (b & c);
    const std::uint32_t second = big0 + majority;
    h = g;
    g = f;
    f = e;
    e = d + first;
    d = c;
    c = b;
    b = a;
    a = first + second;
  }
  h_[0] += a;
  h_[1] += b;
  h_[2] += c;
  h_[3] += d;
  h_[4] += e;
  h_[5] += f;
  h_[6] += g;
  h_[7] += h;
}

void Sha256Stream::feed(std::span<const std::byte> bytes) noexcept {
  total_size_ += bytes.size();
  const std::byte* cursor = bytes.data();
  std::size_t left = bytes.size();
  if (partial_size_) {
    const std::size_t take = std::min(left, sizeof(partial_) - partial_size_);
    std::memcpy(partial_ + partial_size_, cursor, take);
    partial_size_ += take;
    cursor += take;
    left -= take;
    if (partial_size_ < sizeof(partial_)) return;
    block(partial_);
    partial_size_ = 0;
  }
#if defined(__x86_64__)
  if (accelerated_ && left >= 64) {
    const std::size_t whole = left / 64;
    blocks_sha_ni(h_, cursor, whole);
    cursor += whole * 64;
    left -= whole * 64;
  }
#endif
  for (; left >= 64; cursor += 64, left -= 64) block(cursor);
  if (left) std::memcpy(partial_, cursor, left);
  partial_size_ = left;
}

Sha256Digest Sha256Stream::digest() noexcept {
  const std::uint64_t message_bits = total_size_ * 8U;
  // 0x80, zeros up to 56 mod 64, then the bit length, big endian
  partial_[partial_size_++] = std::byte{0x80};
  if (partial_size_ > 56) {
    std::memset(partial_ + partial_size_, 0, 64 - partial_size_);
    block(partial_);
    partial_size_ = 0;
  }
  std::memset(partial_ + partial_size_, 0, 56 - partial_size_);
  for (int index = 0; index < 8; ++index)
    partial_[56 + index] =
        static_cast<std::byte>((message_bits >> (8 * (7 - index))) & 0xffU);
  block(partial_);
  Sha256Digest result;
  for (int word = 0; word < 8; ++word)
    for (int index = 0; index < 4; ++index)
      result[4 * word + index] =
          static_cast<std::byte>((h_[word] >> (8 * (3 - index))) & 0xffU);
  return result;
}

Sha256Digest sha256(std::span<const std::byte> input) noexcept {
  Sha256Stream stream;
  stream.feed(input);
  return stream.digest();
}

Sha256Digest sha256_portable(std::span<const std::byte> input) noexcept {
  Sha256Stream stream(true);
  stream.feed(input);
  return stream.digest();
}

bool constant_time_equal(const Sha256Digest& left,
                         const Sha256Digest& right) noexcept {
  unsigned difference = 0;
  for (std::size_t index = 0; index < left.size(); ++index)
    difference |= std::to_integer<unsigned>(left[index] ^ right[index]);
  return difference == 0;
}

}  // namespace expert::runtime
