// Test infrastructure: C entry points over the hash functions the reference
// itself ships as plain C++ (third_party/column-io/cc/column-io/dataset/
// farmhash.cc and hash_utils.cc), compiled from where they lie by
// oracle/ref_build.sh into oracle/_ref/. Used only to validate the oracle's own
// restatement of FarmHash64 / MurmurHash64A on strings of every length class.
#include <cstddef>
#include <cstdint>

#include "farmhash.h"
#include "hash_utils.h"

extern "C" {

__attribute__((visibility("default"))) uint64_t ref_farm_fingerprint64(const char* s, size_t n) {
  return ::util::Fingerprint64(s, n);
}

__attribute__((visibility("default"))) uint64_t ref_murmur64(const char* s, size_t n, uint64_t seed) {
  return ::column::dataset::MurMurHash64(s, n, seed);
}
}
