// Reader for .npz weight files (the on-disk format of the reference's C++ model and of
// from_npz; the reference reads them with the cnpy library, loaders/npz_load.h:23-75).
// An .npz is a ZIP archive of .npy members: stored (numpy.savez) or deflated (numpy.savez_compressed,
// what the reference's converter writes), with ZIP64 sizes where needed.  Supports little-endian float32,
// float16 and int64 arrays in C order.
#pragma once

#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace turbo_transformers {
namespace loaders {

struct NpyArray {
  std::vector<int64_t> shape;
  char kind = 'f';      // 'f' float, 'i' signed int
  int word_size = 4;    // bytes per element
  std::vector<char> bytes;
  int64_t numel() const {
    int64_t n = 1;
    for (auto d : shape) n *= d;
    return n;
  }
};

// name (without the ".npy" suffix) -> array.  Throws core::EnforceNotMet on malformed input,
// other compression methods or unsupported dtypes.
std::map<std::string, NpyArray> LoadNpz(const std::string& filename);

}  // namespace loaders
}  // namespace turbo_transformers
