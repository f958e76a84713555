// Tensor storage behind the operator graph (reference: src/memory/alloc.hh:9-14,
// src/memory/copy.hh:8-18).  In GPU mode the calls go through the C ABI (dh_pool_alloc, dh_pool_free:
// blocks of a pooled allocator, so lowering operators again makes no hipMalloc; dh_memcpy_*, dh_memset0) and a failing HIP call surfaces as std::runtime_error, the reference's
// convention (src/memory/alloc.cu:6-14); in the CPU modes tensors are plain host arrays.
#pragma once

#include <cstddef>

#include "types.hh"

dbl_t* tensor_alloc(std::size_t size);
void tensor_free(dbl_t* ptr);

// dst is a tensor of the current mode, src a host array (and the reverse for tensor_read).
void tensor_write(dbl_t* dst_begin, dbl_t* dst_end, const dbl_t* src_host);
void tensor_read(const dbl_t* src_begin, const dbl_t* src_end, dbl_t* dst_host);
void tensor_fill(dbl_t* begin, dbl_t* end, dbl_t val);

// Turns a non-zero C-ABI return code into std::runtime_error carrying dh_last_error().
void hip_check(int rc, const char* what);
