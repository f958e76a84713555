#include "images.hh"

#include <cstdio>
#include <memory>
#include <stdexcept>

namespace images
{
namespace
{
using File = std::unique_ptr<std::FILE, int (*)(std::FILE*)>;

// next unsigned integer of a PPM header, skipping white space and '#' comments
std::size_t header_number(std::FILE* f, const std::string& path)
{
    int c = std::fgetc(f);
    for (;;)
    {
        while (c == ' ' || c == '\t' || c == '\n' || c == '\r')
            c = std::fgetc(f);
        if (c != '#')
            break;
        while (c != '\n' && c != EOF)
            c = std::fgetc(f);
    }
    if (c < '0' || c > '9')
        throw std::runtime_error("ppm: malformed header in " + path);
    std::size_t v = 0;
    while (c >= '0' && c <= '9')
    {
        v = v * 10 + (std::size_t)(c - '0');
        c = std::fgetc(f);
    }
    return v;   // the single white-space character after the number has been consumed
}
}  // namespace

void normalize(const std::uint8_t* pix, std::size_t count, dbl_t* out)
{
    for (std::size_t j = 0; j < count; ++j)
        out[j] = dbl_t(pix[j]) / 127.5 - 1.;
}

std::vector<std::uint8_t> load_ppm(const std::string& path, std::size_t* width, std::size_t* height)
{
    File f(std::fopen(path.c_str(), "rb"), std::fclose);
    if (!f)
        throw std::runtime_error("ppm: cannot open " + path);
    if (std::fgetc(f.get()) != 'P' || std::fgetc(f.get()) != '6')
        throw std::runtime_error("ppm: " + path + " is not a binary PPM (P6)");
    const std::size_t w = header_number(f.get(), path), h = header_number(f.get(), path);
    const std::size_t maxval = header_number(f.get(), path);
    if (maxval != 255 || w == 0 || h == 0)
        throw std::runtime_error("ppm: " + path + " must have 8-bit channels and a non-empty size");
    std::vector<std::uint8_t> pix(w * h * 3);
    if (std::fread(pix.data(), 1, pix.size(), f.get()) != pix.size())
        throw std::runtime_error("ppm: truncated file " + path);
    if (width) *width = w;
    if (height) *height = h;
    return pix;
}

void save_ppm(const std::string& path, const std::uint8_t* pix, std::size_t width, std::size_t height)
{
    File f(std::fopen(path.c_str(), "wb"), std::fclose);
    if (!f)
        throw std::runtime_error("ppm: cannot open " + path + " for writing");
    std::fprintf(f.get(), "P6\n%zu %zu\n255\n", width, height);
    if (std::fwrite(pix, 1, width * height * 3, f.get()) != width * height * 3)
        throw std::runtime_error("ppm: write failed for " + path);
}

std::vector<dbl_t> load(const std::string& dir, const std::vector<std::size_t>& idxs)
{
    std::vector<dbl_t> res(IMG_SIZE * idxs.size());
    for (std::size_t i = 0; i < idxs.size(); ++i)
    {
        std::string idx = std::to_string(idxs[i]);
        while (idx.size() < 6)
            idx = "0" + idx;
        const std::string path = dir + (dir.empty() || dir.back() == '/' ? "" : "/") + idx + ".ppm";
        std::size_t w = 0, h = 0;
        const std::vector<std::uint8_t> pix = load_ppm(path, &w, &h);
        if (w != IMG_SIDE || h != IMG_SIDE)
            throw std::runtime_error("images::load: " + path + " is not 64x64");
        normalize(pix.data(), IMG_SIZE, res.data() + i * IMG_SIZE);
    }
    return res;
}

std::vector<dbl_t> load(const std::string& dir, std::size_t idx_beg, std::size_t idx_end)
{
    std::vector<std::size_t> idxs;
    for (std::size_t i = idx_beg; i < idx_end; ++i)
        idxs.push_back(i);
    return load(dir, idxs);
}

void save_samples(const dbl_t* data, std::size_t width, std::size_t height, const std::string& path)
{
    std::vector<std::uint8_t> pixs(width * height * IMG_SIZE);
    for (std::size_t i = 0; i < width; ++i)
        for (std::size_t j = 0; j < height; ++j)
        {
            const dbl_t* img = data + (j * width + i) * IMG_SIZE;
            const std::size_t out_x = i * IMG_SIDE, out_y = j * IMG_SIDE;
            for (std::size_t y = 0; y < IMG_SIDE; ++y)
                for (std::size_t x = 0; x < IMG_SIDE; ++x)
                    for (std::size_t c = 0; c < 3; ++c)
                    {
                        const double v = (img[y * IMG_SIDE * 3 + x * 3 + c] + 1.) * 127.5;
                        pixs[(out_y + y) * (width * IMG_SIDE * 3) + (out_x + x) * 3 + c] =
                            v <= 0. ? 0 : v >= 255. ? 255 : (std::uint8_t)v;
                    }
        }
    save_ppm(path, pixs.data(), width * IMG_SIDE, height * IMG_SIDE);
}

}  // namespace images
