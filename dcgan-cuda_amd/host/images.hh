// Image batches in and sample mosaics out, as the reference's celebA helpers do
// (src/datasets/celeba.cu:16-68), with binary PPM (P6) files in place of JPEG: the reference decodes
// and encodes through libjpeg, which is outside this build.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "types.hh"

namespace images
{

constexpr std::size_t IMG_SIDE = 64;
constexpr std::size_t IMG_SIZE = IMG_SIDE * IMG_SIDE * 3;

// out[j] = pix[j] / 127.5 - 1, evaluated in double as the reference's expression is
// (src/datasets/celeba.cu:27-28).
void normalize(const std::uint8_t* pix, std::size_t count, dbl_t* out);

// Reads / writes an 8-bit RGB image as binary PPM.
std::vector<std::uint8_t> load_ppm(const std::string& path, std::size_t* width, std::size_t* height);
void save_ppm(const std::string& path, const std::uint8_t* pix, std::size_t width, std::size_t height);

// Images <dir>/<6-digit index>.ppm (64x64 RGB) as one normalised batch [idxs.size(), 64, 64, 3]
// (src/datasets/celeba.cu:16-34 with .ppm in place of .jpg).
std::vector<dbl_t> load(const std::string& dir, const std::vector<std::size_t>& idxs);
std::vector<dbl_t> load(const std::string& dir, std::size_t idx_beg, std::size_t idx_end);

// width x height images [.., 64, 64, 3] in [-1, 1] as one mosaic, image (j * width + i) at column i,
// row j; pixel = (v + 1) * 127.5 truncated (src/datasets/celeba.cu:44-68).  Values outside [-1, 1]
// are clamped to 0 / 255 (the reference's conversion is undefined for them).
void save_samples(const dbl_t* data, std::size_t width, std::size_t height, const std::string& path);

}  // namespace images
