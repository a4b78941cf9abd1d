// 128-bit content hash of host memory, for the prepared-weight cache of tnns_conv (ftnn_api.hip): the cache finds a
// layer's weights again by what they contain, so the hash is recomputed on every call and must cost less than the
// upload it saves.  Host code only.
//
// Two implementations with the same interface, chosen once at run time:
//   * AES rounds (x86 with AES-NI): four independent 128-bit lanes, one AESENC per 16 bytes, 64 bytes per trip;
//     limited by memory, not by the arithmetic;
//   * multiply-rotate lanes over 32-byte blocks (any CPU).
// Not cryptographic: it guards against a caller rewriting or re-packing weights, not against an adversary.  Both
// halves of the result depend on every input byte and on the length.
#include "host_hash.h"

#include <string.h>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

namespace ftnn {

namespace {

inline uint64_t rotl(uint64_t v, int r) { return (v << r) | (v >> (64 - r)); }

inline uint64_t fmix(uint64_t h) {
    h ^= h >> 33;
    h *= 0xFF51AFD7ED558CCDull;
    h ^= h >> 29;
    h *= 0xC4CEB9FE1A85EC53ull;
    h ^= h >> 32;
    return h;
}

Hash128 hash_portable(const void* data, size_t bytes, uint64_t seed) {
    const unsigned char* p = static_cast<const unsigned char*>(data);
    uint64_t h0 = 0x9E3779B97F4A7C15ull ^ seed, h1 = 0xC2B2AE3D27D4EB4Full + seed, h2 = 0x165667B19E3779F9ull ^ rotl(seed, 21),
             h3 = 0x27D4EB2F165667C5ull + rotl(seed, 43);
    const size_t blocks = bytes / 32;
    for (size_t i = 0; i < blocks; i++, p += 32) {
        uint64_t w[4];
        memcpy(w, p, 32);
        h0 = rotl((h0 ^ w[0]) * 0xFF51AFD7ED558CCDull, 29);
        h1 = rotl((h1 ^ w[1]) * 0xC4CEB9FE1A85EC53ull, 31);
        h2 = rotl((h2 ^ w[2]) * 0x9FB21C651E98DF25ull, 27);
        h3 = rotl((h3 ^ w[3]) * 0xD6E8FEB86659FD93ull, 33);
    }
    for (size_t i = 0; i < bytes % 32; i++) h0 = rotl((h0 ^ p[i]) * 0xFF51AFD7ED558CCDull, 29);
    Hash128 out;
    out.lo = fmix(h0 ^ rotl(h1, 17) ^ rotl(h2, 34) ^ rotl(h3, 51) ^ (uint64_t)bytes);
    out.hi = fmix((h0 + rotl(h2, 13)) ^ (rotl(h1, 41) + h3) ^ ((uint64_t)bytes * 0x9E3779B97F4A7C15ull));
    return out;
}

#if defined(__x86_64__)
__attribute__((target("aes,sse4.1"))) Hash128 hash_aes(const void* data, size_t bytes, uint64_t seed) {
    const unsigned char* p = static_cast<const unsigned char*>(data);
    const __m128i k0 = _mm_set_epi64x((long long)0x9E3779B97F4A7C15ull, (long long)0xC2B2AE3D27D4EB4Full);
    const __m128i k1 = _mm_set_epi64x((long long)0x165667B19E3779F9ull, (long long)0x27D4EB2F165667C5ull);
    const __m128i k2 = _mm_set_epi64x((long long)0xFF51AFD7ED558CCDull, (long long)0xC4CEB9FE1A85EC53ull);
    const __m128i k3 = _mm_set_epi64x((long long)0x9FB21C651E98DF25ull, (long long)0xD6E8FEB86659FD93ull);
    const __m128i sd = _mm_set_epi64x((long long)seed, (long long)~seed);
    __m128i s0 = _mm_xor_si128(k0, sd), s1 = _mm_xor_si128(k1, sd), s2 = _mm_xor_si128(k2, sd), s3 = _mm_xor_si128(k3, sd);
    size_t left = bytes;
    for (; left >= 64; left -= 64, p += 64) {
        // state <- AESENC(state xor block, key): the block passes through SubBytes / ShiftRows / MixColumns
        s0 = _mm_aesenc_si128(_mm_xor_si128(s0, _mm_loadu_si128(reinterpret_cast<const __m128i*>(p))), k0);
        s1 = _mm_aesenc_si128(_mm_xor_si128(s1, _mm_loadu_si128(reinterpret_cast<const __m128i*>(p + 16))), k1);
        s2 = _mm_aesenc_si128(_mm_xor_si128(s2, _mm_loadu_si128(reinterpret_cast<const __m128i*>(p + 32))), k2);
        s3 = _mm_aesenc_si128(_mm_xor_si128(s3, _mm_loadu_si128(reinterpret_cast<const __m128i*>(p + 48))), k3);
    }
    if (left) {   // the last partial block, zero-padded (the length enters below)
        unsigned char tail[64] = {0};
        memcpy(tail, p, left);
        s0 = _mm_aesenc_si128(_mm_xor_si128(s0, _mm_loadu_si128(reinterpret_cast<const __m128i*>(tail))), k0);
        s1 = _mm_aesenc_si128(_mm_xor_si128(s1, _mm_loadu_si128(reinterpret_cast<const __m128i*>(tail + 16))), k1);
        s2 = _mm_aesenc_si128(_mm_xor_si128(s2, _mm_loadu_si128(reinterpret_cast<const __m128i*>(tail + 32))), k2);
        s3 = _mm_aesenc_si128(_mm_xor_si128(s3, _mm_loadu_si128(reinterpret_cast<const __m128i*>(tail + 48))), k3);
    }
    // fold the lanes with further rounds so that every output bit depends on every lane, then the length
    const __m128i len = _mm_set_epi64x((long long)bytes, (long long)(bytes * 0x9E3779B97F4A7C15ull));
    __m128i a = _mm_aesenc_si128(_mm_xor_si128(s0, len), s1);
    __m128i b = _mm_aesenc_si128(_mm_xor_si128(s2, len), s3);
    a = _mm_aesenc_si128(a, b);
    b = _mm_aesenc_si128(b, k2);
    a = _mm_aesenc_si128(_mm_xor_si128(a, b), k0);
    a = _mm_aesenc_si128(a, k1);
    a = _mm_aesenc_si128(a, k3);
    Hash128 out;
    out.lo = (uint64_t)_mm_cvtsi128_si64(a);
    out.hi = (uint64_t)_mm_extract_epi64(a, 1);
    return out;
}
#endif

}  // namespace

bool hash128_uses_aes() {
#if defined(__x86_64__)
    static const bool yes = __builtin_cpu_supports("aes") && __builtin_cpu_supports("sse4.1");
    return yes;
#else
    return false;
#endif
}

Hash128 hash128(const void* data, size_t bytes, uint64_t seed) {
#if defined(__x86_64__)
    if (hash128_uses_aes()) return hash_aes(data, bytes, seed);
#endif
    return hash_portable(data, bytes, seed);
}

Hash128 hash128_portable(const void* data, size_t bytes, uint64_t seed) { return hash_portable(data, bytes, seed); }

}  // namespace ftnn
