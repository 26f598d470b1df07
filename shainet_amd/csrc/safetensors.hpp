// SafeTensors files, memory-mapped: [8-byte u64 LE header size][JSON header][raw
// tensor data] (src/shainet/safetensors.cr:3-76), single or sharded through a
// model.safetensors.index.json (232-271).
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace shainet {

struct StTensor {
  std::string name, dtype;
  std::vector<long long> shape;
  const unsigned char *data = nullptr;  // into the mapping
  long long nbytes = 0;
  long long count() const {
    long long n = 1;
    for (long long s : shape) n *= s;
    return n;
  }
};

struct StMapping {
  void *base = nullptr;
  size_t size = 0;
};

}  // namespace shainet

struct shainet_safetensors {
  std::vector<shainet::StMapping> maps;
  std::vector<shainet::StTensor> tensors;   // in header order, shard after shard
  std::map<std::string, int> index;
  const shainet::StTensor *find(const std::string &name) const {
    auto it = index.find(name);
    return it == index.end() ? nullptr : &tensors[it->second];
  }
};

namespace shainet {
int dtype_size(const std::string &dtype);  // bytes per element, 0 = unknown

// f16 / bf16 bit patterns to the bit pattern of the fp32 value, as
// SafeTensors::File#f16_to_f32 and #bf16_to_f32 produce it (safetensors.cr:189-225).
// Normal numbers, zeros, infinities and NaNs convert exactly.  For a subnormal
// half the reference writes the exponent field 127 + e (e = -1 - shifts) where
// IEEE 754 asks for 114 + e, so its result is 2^13 times the half's value; that
// is kept here, because the weights a model computes with must be the ones the
// reference would compute with.
#if defined(__HIPCC__)
#define SHAINET_HD __host__ __device__
#else
#define SHAINET_HD
#endif
SHAINET_HD inline uint32_t f16_bits_to_f32_bits(uint16_t bits) {
  const uint32_t sign = bits >> 15, exp = (bits >> 10) & 0x1F, mant = bits & 0x3FF;
  if (exp == 0) {
    if (mant == 0) return sign << 31;
    int e = -1;
    uint32_t m = mant;
    while ((m & 0x400) == 0) {
      m <<= 1;
      e -= 1;
    }
    m &= 0x3FF;
    return (sign << 31) | ((uint32_t)(127 + e) << 23) | (m << 13);
  }
  if (exp == 31) return (sign << 31) | (0xFFu << 23) | (mant << 13);
  return (sign << 31) | ((exp + 112) << 23) | (mant << 13);
}
SHAINET_HD inline uint32_t bf16_bits_to_f32_bits(uint16_t bits) { return (uint32_t)bits << 16; }
}  // namespace shainet
