// Minimal reader / writer of numpy's .npz container (a ZIP archive of .npy members) for float
// tensors, so that weights can be exchanged with numpy directly.  The reference stores its weights
// through the external tocha library (`tbin` files converted from .npz by a tool of that library,
// src/ops/graph.cu:326-361); this build reads and writes the .npz itself.
//
// Supported: members stored without compression (what numpy.savez writes), little-endian float32 or
// float64 data in C order, archives below 4 GiB.  Anything else raises std::runtime_error.
#pragma once

#include <cstddef>
#include <string>
#include <vector>

namespace npz
{

struct Array
{
    std::string name;              // member name without the ".npy" suffix
    std::vector<std::size_t> shape;
    std::vector<float> data;       // row-major
    std::size_t size() const;
};

void save(const std::string& path, const std::vector<Array>& arrays);
std::vector<Array> load(const std::string& path);

}  // namespace npz
