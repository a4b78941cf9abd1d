// 128-bit content hash of host memory (host_hash.cpp): identity of a layer's packed weights in the prepared-weight
// cache of the host entry points.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace ftnn {

struct Hash128 {
    uint64_t lo, hi;
    bool operator==(const Hash128& o) const { return lo == o.lo && hi == o.hi; }
};

// hash of bytes [data, data + bytes) under `seed`; AES rounds where the CPU has them, multiply-rotate lanes otherwise
Hash128 hash128(const void* data, size_t bytes, uint64_t seed);
// the portable implementation whatever the CPU (for tests of both)
Hash128 hash128_portable(const void* data, size_t bytes, uint64_t seed);
bool hash128_uses_aes();

}  // namespace ftnn
