#include "npz.hh"

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <stdexcept>

namespace npz
{
namespace
{

[[noreturn]] void bad(const std::string& path, const std::string& what)
{
    throw std::runtime_error("npz: " + path + ": " + what);
}

std::uint32_t crc32(const unsigned char* p, std::size_t n, std::uint32_t crc = 0)
{
    static std::uint32_t table[256];
    static bool ready = false;
    if (!ready)
    {
        for (std::uint32_t i = 0; i < 256; ++i)
        {
            std::uint32_t c = i;
            for (int k = 0; k < 8; ++k)
                c = (c & 1) ? 0xEDB88320u ^ (c >> 1) : c >> 1;
            table[i] = c;
        }
        ready = true;
    }
    crc = ~crc;
    for (std::size_t i = 0; i < n; ++i)
        crc = table[(crc ^ p[i]) & 0xff] ^ (crc >> 8);
    return ~crc;
}

void put16(std::string& s, std::uint16_t v) { s.push_back((char)(v & 0xff)); s.push_back((char)(v >> 8)); }
void put32(std::string& s, std::uint32_t v) { put16(s, (std::uint16_t)(v & 0xffff)); put16(s, (std::uint16_t)(v >> 16)); }
std::uint16_t get16(const unsigned char* p) { return (std::uint16_t)(p[0] | (p[1] << 8)); }
std::uint32_t get32(const unsigned char* p) { return get16(p) | ((std::uint32_t)get16(p + 2) << 16); }

// .npy version 1.0 header for a C-ordered little-endian float32 array; the data starts 64-byte aligned
std::string npy_header(const std::vector<std::size_t>& shape)
{
    std::string dict = "{'descr': '<f4', 'fortran_order': False, 'shape': (";
    for (std::size_t i = 0; i < shape.size(); ++i)
        dict += std::to_string(shape[i]) + (shape.size() == 1 || i + 1 < shape.size() ? "," : "") +
                (i + 1 < shape.size() ? " " : "");
    dict += "), }";
    std::size_t total = 10 + dict.size() + 1;
    dict.append((64 - total % 64) % 64, ' ');
    dict.push_back('\n');
    std::string h("\x93NUMPY\x01\x00", 8);
    put16(h, (std::uint16_t)dict.size());
    return h + dict;
}

}  // namespace

std::size_t Array::size() const
{
    std::size_t n = 1;
    for (std::size_t d : shape)
        n *= d;
    return n;
}

void save(const std::string& path, const std::vector<Array>& arrays)
{
    std::FILE* f = std::fopen(path.c_str(), "wb");
    if (!f)
        bad(path, "cannot open for writing");
    std::unique_ptr<std::FILE, int (*)(std::FILE*)> guard(f, std::fclose);
    std::string central;
    std::uint64_t offset = 0;
    for (const Array& a : arrays)
    {
        if (a.data.size() != a.size())
            bad(path, "array '" + a.name + "' has " + std::to_string(a.data.size()) + " values for its shape");
        const std::string member = a.name + ".npy";
        const std::string header = npy_header(a.shape);
        const std::uint64_t bytes = header.size() + a.data.size() * sizeof(float);
        if (offset + bytes + member.size() + 30 >= 0xffffffffull)
            bad(path, "archives of 4 GiB and more are not supported");
        std::uint32_t crc = crc32(reinterpret_cast<const unsigned char*>(header.data()), header.size());
        crc = crc32(reinterpret_cast<const unsigned char*>(a.data.data()), a.data.size() * sizeof(float), crc);
        std::string local;
        put32(local, 0x04034b50); put16(local, 20); put16(local, 0); put16(local, 0);   // version, flags, stored
        put16(local, 0); put16(local, 0x21);                                           // time, date (1980-01-01)
        put32(local, crc); put32(local, (std::uint32_t)bytes); put32(local, (std::uint32_t)bytes);
        put16(local, (std::uint16_t)member.size()); put16(local, 0);
        local += member;
        put32(central, 0x02014b50); put16(central, 20); put16(central, 20); put16(central, 0); put16(central, 0);
        put16(central, 0); put16(central, 0x21);
        put32(central, crc); put32(central, (std::uint32_t)bytes); put32(central, (std::uint32_t)bytes);
        put16(central, (std::uint16_t)member.size()); put16(central, 0); put16(central, 0);   // name, extra, comment
        put16(central, 0); put16(central, 0); put32(central, 0);                              // disk, attributes
        put32(central, (std::uint32_t)offset);
        central += member;
        if (std::fwrite(local.data(), 1, local.size(), f) != local.size() ||
            std::fwrite(header.data(), 1, header.size(), f) != header.size() ||
            std::fwrite(a.data.data(), sizeof(float), a.data.size(), f) != a.data.size())
            bad(path, "write failed");
        offset += local.size() + bytes;
    }
    std::string end;
    put32(end, 0x06054b50); put16(end, 0); put16(end, 0);
    put16(end, (std::uint16_t)arrays.size()); put16(end, (std::uint16_t)arrays.size());
    put32(end, (std::uint32_t)central.size()); put32(end, (std::uint32_t)offset); put16(end, 0);
    if (arrays.size() > 0xfffe)
        bad(path, "too many arrays");
    if (std::fwrite(central.data(), 1, central.size(), f) != central.size() ||
        std::fwrite(end.data(), 1, end.size(), f) != end.size())
        bad(path, "write failed");
}

std::vector<Array> load(const std::string& path)
{
    std::FILE* f = std::fopen(path.c_str(), "rb");
    if (!f)
        bad(path, "cannot open");
    std::unique_ptr<std::FILE, int (*)(std::FILE*)> guard(f, std::fclose);
    std::fseek(f, 0, SEEK_END);
    const long file_size = std::ftell(f);
    if (file_size < 22)
        bad(path, "not a zip archive");
    // end-of-central-directory record: in the last 64 KiB + 22 bytes
    const long tail = file_size < 65557 ? file_size : 65557;
    std::vector<unsigned char> buf((std::size_t)tail);
    std::fseek(f, file_size - tail, SEEK_SET);
    if (std::fread(buf.data(), 1, buf.size(), f) != buf.size())
        bad(path, "read failed");
    long eocd = -1;
    for (long i = tail - 22; i >= 0; --i)
        if (get32(&buf[(std::size_t)i]) == 0x06054b50)
        {
            eocd = i;
            break;
        }
    if (eocd < 0)
        bad(path, "no zip end record");
    const std::uint32_t count = get16(&buf[(std::size_t)eocd + 10]);
    const std::uint32_t cd_size = get32(&buf[(std::size_t)eocd + 12]);
    const std::uint32_t cd_off = get32(&buf[(std::size_t)eocd + 16]);
    if (count == 0xffff || cd_off == 0xffffffffu)
        bad(path, "zip64 archives are not supported");
    if ((std::uint64_t)cd_off + cd_size > (std::uint64_t)file_size)
        bad(path, "central directory lies outside the file");
    std::vector<unsigned char> cd(cd_size);
    std::fseek(f, (long)cd_off, SEEK_SET);
    if (std::fread(cd.data(), 1, cd.size(), f) != cd.size())
        bad(path, "truncated central directory");
    std::vector<Array> out;
    std::size_t at = 0;
    for (std::uint32_t e = 0; e < count; ++e)
    {
        if (at + 46 > cd.size() || get32(&cd[at]) != 0x02014b50)
            bad(path, "corrupt central directory");
        const std::uint16_t method = get16(&cd[at + 10]);
        const std::uint32_t csize = get32(&cd[at + 20]), usize = get32(&cd[at + 24]);
        const std::uint16_t nlen = get16(&cd[at + 28]), xlen = get16(&cd[at + 30]), clen = get16(&cd[at + 32]);
        const std::uint32_t local_off = get32(&cd[at + 42]);
        if (at + 46 + (std::size_t)nlen + xlen + clen > cd.size())
            bad(path, "corrupt central directory (entry runs past its end)");
        std::string member(reinterpret_cast<const char*>(&cd[at + 46]), nlen);
        at += 46 + (std::size_t)nlen + xlen + clen;
        if (method != 0)
            bad(path, "member '" + member + "' is compressed; write the file with numpy.savez, not savez_compressed");
        if (csize == 0xffffffffu || usize == 0xffffffffu || local_off == 0xffffffffu)
            bad(path, "member '" + member + "' needs zip64, which is not supported");
        if (csize != usize)
            bad(path, "member '" + member + "': stored and original sizes differ");
        unsigned char lh[30];
        if ((std::uint64_t)local_off + 30 > (std::uint64_t)file_size)
            bad(path, "member '" + member + "' lies outside the file");
        std::fseek(f, (long)local_off, SEEK_SET);
        if (std::fread(lh, 1, 30, f) != 30 || get32(lh) != 0x04034b50)
            bad(path, "corrupt local header of '" + member + "'");
        const std::uint64_t data_off = (std::uint64_t)local_off + 30 + get16(lh + 26) + get16(lh + 28);
        if (data_off + usize > (std::uint64_t)file_size)
            bad(path, "truncated member '" + member + "'");
        std::vector<unsigned char> raw(usize);
        std::fseek(f, (long)data_off, SEEK_SET);
        if (std::fread(raw.data(), 1, raw.size(), f) != raw.size())
            bad(path, "truncated member '" + member + "'");
        // .npy: magic, version, header length (2 bytes for v1, 4 for v2/3), python dict literal
        if (raw.size() < 10 || std::memcmp(raw.data(), "\x93NUMPY", 6) != 0)
            bad(path, "member '" + member + "' is not a .npy array");
        const int major = raw[6];
        std::size_t hlen, hstart;
        if (major == 1) { hlen = get16(&raw[8]); hstart = 10; }
        else { if (raw.size() < 12) bad(path, "short .npy header"); hlen = get32(&raw[8]); hstart = 12; }
        if (hstart + hlen > raw.size())
            bad(path, "short .npy header in '" + member + "'");
        const std::string dict(reinterpret_cast<const char*>(&raw[hstart]), hlen);
        auto value_after = [&](const std::string& key) {
            const std::size_t k = dict.find("'" + key + "'");
            if (k == std::string::npos)
                bad(path, "'" + member + "': no " + key + " in the .npy header");
            const std::size_t colon = dict.find(':', k);
            if (colon == std::string::npos)
                bad(path, "'" + member + "': malformed " + key + " in the .npy header");
            return colon + 1;
        };
        const std::size_t d0 = dict.find('\'', value_after("descr"));
        const std::size_t d1 = d0 == std::string::npos ? d0 : dict.find('\'', d0 + 1);
        if (d1 == std::string::npos)
            bad(path, "'" + member + "': malformed descr in the .npy header");
        const std::string descr = dict.substr(d0 + 1, d1 - d0 - 1);
        if (descr != "<f4" && descr != "<f8")
            bad(path, "'" + member + "' has dtype " + descr + "; float32 or float64 expected");
        const std::size_t fo = dict.find_first_not_of(' ', value_after("fortran_order"));
        if (fo == std::string::npos || dict.compare(fo, 5, "False") != 0)
            bad(path, "'" + member + "' is in Fortran order");
        Array a;
        a.name = member.size() > 4 && member.compare(member.size() - 4, 4, ".npy") == 0
                     ? member.substr(0, member.size() - 4) : member;
        const std::size_t s0 = dict.find('(', value_after("shape"));
        const std::size_t s1 = s0 == std::string::npos ? s0 : dict.find(')', s0);
        if (s1 == std::string::npos)
            bad(path, "'" + member + "': no shape tuple in the .npy header");
        const std::size_t esz = descr == "<f4" ? 4 : 8, payload = raw.size() - hstart - hlen;
        std::size_t num = 0, n = 1;
        bool in_num = false;
        for (std::size_t i = s0 + 1; i <= s1; ++i)
        {
            const char c = dict[i];
            if (c >= '0' && c <= '9')
            {
                if (num > payload)   // no dimension can exceed the payload: stops the digits from wrapping
                    bad(path, "'" + member + "': data size does not match its shape");
                num = num * 10 + (std::size_t)(c - '0');
                in_num = true;
            }
            else if (in_num)
            {
                // the element count stays within the payload, so neither it nor n * esz can wrap
                if (num != 0 && n > payload / num)
                    bad(path, "'" + member + "': data size does not match its shape");
                n *= num;
                a.shape.push_back(num);
                num = 0;
                in_num = false;
            }
        }
        if (n > payload / esz || n * esz != payload)
            bad(path, "'" + member + "': data size does not match its shape");
        a.data.resize(n);
        const unsigned char* src = &raw[hstart + hlen];
        if (esz == 4)
            std::memcpy(a.data.data(), src, n * 4);
        else
            for (std::size_t i = 0; i < n; ++i)
            {
                double d;
                std::memcpy(&d, src + 8 * i, 8);
                a.data[i] = (float)d;
            }
        out.push_back(std::move(a));
    }
    return out;
}

}  // namespace npz
