#include "memory.hh"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "dcgan_hip.h"
#include "mode.hh"

namespace
{
bool g_mode_known = false;
ProgramMode g_mode = ProgramMode::MONOTHREAD;
}  // namespace

ProgramMode program_mode()
{
    if (!g_mode_known)
    {
        const char* env = std::getenv("RT_MODE");
        g_mode = ProgramMode::MONOTHREAD;
        if (env && !std::strcmp(env, "GPU"))
            g_mode = ProgramMode::GPU;
        else if (env && !std::strcmp(env, "MCPU"))
            g_mode = ProgramMode::MULTITHREAD;
        g_mode_known = true;
    }
    return g_mode;
}

void program_mode_reset()
{
    g_mode_known = false;
}

void hip_check(int rc, const char* what)
{
    if (rc != 0)
        throw std::runtime_error(std::string(what) + ": " + dh_last_error());
}

dbl_t* tensor_alloc(std::size_t size)
{
    if (program_mode() == ProgramMode::GPU)
    {
        void* p = nullptr;
        hip_check(dh_pool_alloc(&p, size * sizeof(dbl_t)), "tensor_alloc");
        return static_cast<dbl_t*>(p);
    }
    return new dbl_t[size];
}

void tensor_free(dbl_t* ptr)
{
    if (program_mode() == ProgramMode::GPU)
        hip_check(dh_pool_free(ptr), "tensor_free");
    else
        delete[] ptr;
}

void tensor_write(dbl_t* dst_begin, dbl_t* dst_end, const dbl_t* src_host)
{
    const std::size_t n = dst_end - dst_begin;
    if (program_mode() == ProgramMode::GPU)
        // stream-ordered behind the work already queued (every instruction runs on the default stream):
        // the caller's buffer is free on return, and a run that is still executing is not waited for
        hip_check(dh_memcpy_h2d_staged(dst_begin, src_host, n * sizeof(dbl_t), nullptr), "tensor_write");
    else
        std::copy(src_host, src_host + n, dst_begin);
}

void tensor_read(const dbl_t* src_begin, const dbl_t* src_end, dbl_t* dst_host)
{
    const std::size_t n = src_end - src_begin;
    if (program_mode() == ProgramMode::GPU)
        hip_check(dh_memcpy_d2h(dst_host, src_begin, n * sizeof(dbl_t)), "tensor_read");
    else
        std::copy(src_begin, src_end, dst_host);
}

void tensor_fill(dbl_t* begin, dbl_t* end, dbl_t val)
{
    const std::size_t n = end - begin;
    if (program_mode() != ProgramMode::GPU)
    {
        std::fill(begin, end, val);
        return;
    }
    if (val == 0)
    {
        hip_check(dh_memset0(begin, n * sizeof(dbl_t), nullptr), "tensor_fill");
        hip_check(dh_sync(), "tensor_fill");
        return;
    }
    std::vector<dbl_t> host(n, val);
    hip_check(dh_memcpy_h2d(begin, host.data(), n * sizeof(dbl_t)), "tensor_fill");
}
