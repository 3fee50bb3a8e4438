// C++ front end of libw4a16.so with the interface of TurboMind's weight-format functions
// (src/turbomind/kernels/gemm_s_f16/format.h:11-30 in lmdeploy): same names, same argument
// order, hipStream_t instead of cudaStream_t.  Errors become std::runtime_error.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <stdexcept>

#include "../w4a16.h"

namespace turbomind {

namespace detail {
inline void w4a16_raise(int rc)
{
    if (rc < 0) throw std::runtime_error(w4a16_last_error());
}
}  // namespace detail

// format.h:15-24.  A_dst comes out in the gfx950 tiled layout (not the reference's), Q_dst is
// bit-identical to the reference's; workspace is unused.
inline void convert_s4_k_m8(uint32_t*       A_dst,
                            half2*          Q_dst,
                            half*           workspace,
                            const uint32_t* A_src,
                            const half*     scales,
                            const uint32_t* qzeros,
                            int             m,
                            int             k,
                            int             group_size,
                            hipStream_t     st = {})
{
    detail::w4a16_raise(w4a16_convert_s4_k_m8(A_dst, Q_dst, workspace, A_src, scales, qzeros, m, k, group_size, (void*)st));
}

// format.h:26
inline void
transpose_qk_s4_k_m8_hf(uint32_t* dst, const uint32_t* src, int m, int k, int size_per_head, hipStream_t st = {})
{
    detail::w4a16_raise(w4a16_transpose_qk_s4_k_m8_hf(dst, src, m, k, size_per_head, (void*)st));
}

// format.h:28
inline void fuse_w1_w3_s4_k_m8(uint32_t* dst, const uint32_t* src, int m, int k, hipStream_t st = {})
{
    detail::w4a16_raise(w4a16_fuse_w1_w3_s4_k_m8(dst, src, m, k, (void*)st));
}

// format.h:30 (dst holds 8 fp16 per source word)
inline void dequantize_s4(uint4* dst, const uint32_t* src, size_t count, hipStream_t st = {})
{
    detail::w4a16_raise(w4a16_dequantize_s4(dst, src, count, (void*)st));
}

// format.h:13: AWQ words -> the tiled weight layout the GEMM reads (here the gfx950 one); the
// weight half of convert_s4_k_m8.
inline void reformat_s4_k_m8(uint32_t* dst, const uint32_t* src, int m, int k, hipStream_t st = {})
{
    detail::w4a16_raise(w4a16_reformat_s4_k_m8(dst, src, m, k, (void*)st));
}

}  // namespace turbomind
