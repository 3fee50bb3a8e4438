// Measurement aids, not part of the GEMM path: plain streaming reads of a buffer, launched like the
// decode kernels.  Their time on a buffer of a matrix's size is the ceiling that launch + first trip
// to HBM + streaming set for any kernel that has to read that matrix once.
//
// probe_read_kernel: the simplest form (compiler-scheduled loop, one 512-thread workgroup per CU and
// pass, four 16-byte non-temporal loads in flight per lane, drained every trip).
// probe_stream_kernel: the form the GEMM kernels use - loads issued from inline assembly in place and
// waited for by count, so that a constant number of them stays in flight per lane from the first
// instruction to the last - with the number in flight, the workgroups per CU and the cache hint as
// parameters, for sweeping what the memory system gives at best.
// probe_mfma_kernel: nothing but v_mfma_f32_16x16x32_f16 on registers, for the rate the matrix pipes reach at
// the clock the chip settles at under them.
#include "w4a16_common.h"

#include <algorithm>
#include <type_traits>

namespace w4a16 {

namespace {

__global__ void __launch_bounds__(512) probe_read_kernel(const u32x4_t* __restrict__ src, size_t vecs, uint32_t* sink)
{
    u32x4_t      acc    = {0, 0, 0, 0};
    const size_t stride = (size_t)gridDim.x * 512 * 4;
    for (size_t i = (size_t)blockIdx.x * 512 * 4 + threadIdx.x; i < vecs; i += stride) {
        // four loads in flight per lane, 8 KiB per wave and trip
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t j = i + (size_t)u * 512;
            if (j < vecs) acc ^= __builtin_nontemporal_load(src + j);
        }
    }
    const uint32_t x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (x == 0x9e3779b9u) sink[blockIdx.x] = x;  // (keeps the loads alive; practically never taken)
}

template<int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// One 16-byte load per lane at sbase + voff, in place; with flag 0 it is issued under EXEC = 0: it
// still counts in vmcnt but touches neither memory nor its destination.
template<int HINT>
__device__ __forceinline__ void probe_load(u32x4_t& dst, uint32_t voff, const void* sbase, bool enable)
{
    uint64_t  sv;
    const int flag = __builtin_amdgcn_readfirstlane(enable ? 1 : 0);
#define W4A16_PROBE_LOAD(hint)                                                                                         \
    asm volatile("s_mov_b64 %[sv], exec\n\ts_cmp_lg_u32 %[mk], 0\n\ts_cselect_b64 exec, exec, 0\n\t"                    \
                 "global_load_dwordx4 %[d], %[vo], %[sb] " hint "\n\ts_mov_b64 exec, %[sv]"                             \
                 : [d] "+v"(dst), [sv] "=&s"(sv)                                                                       \
                 : [vo] "v"(voff), [sb] "s"(sbase), [mk] "s"(flag)                                                     \
                 : "scc")
    if constexpr (HINT == 0) W4A16_PROBE_LOAD("");
    else if constexpr (HINT == 1) W4A16_PROBE_LOAD("nt");
    else W4A16_PROBE_LOAD("sc0 sc1");
#undef W4A16_PROBE_LOAD
}

// Every wave keeps U loads of 1 KiB in flight; block number i of wave w is w + i * (waves of the
// grid), so at any moment the chip reads one contiguous window of the buffer.
template<int U, int HINT>
__global__ void __launch_bounds__(512) probe_stream_kernel(const char* __restrict__ src, int blocks, uint32_t* sink,
                                                           unsigned long long* clk)
{
    clock_record_start(clk, blockIdx.x == gridDim.x / 2 && threadIdx.x == 0);
    const int lane   = threadIdx.x & 63;
    const int wid    = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * 8 + (threadIdx.x >> 6)));
    const int nwaves = gridDim.x * 8;
    const int cnt    = wid < blocks ? (blocks - wid + nwaves - 1) / nwaves : 0;
    const uint32_t voff = (uint32_t)lane * 16;
    u32x4_t r[U];
#pragma unroll
    for (int u = 0; u < U; ++u) r[u] = u32x4_t{0, 0, 0, 0};
    auto base = [&](int i) { return src + (int64_t)(wid + (int64_t)min(i, max(cnt - 1, 0)) * nwaves) * 1024; };
    static_for<0, U>([&](auto u) { probe_load<HINT>(r[decltype(u)::value], voff, base(decltype(u)::value), decltype(u)::value < cnt); });
    u32x4_t acc = {0, 0, 0, 0};
    for (int i = 0; i < cnt; i += U) {
        static_for<0, U>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r[u]) : "n"(U - 1));
            if (i + u < cnt) acc ^= r[u];
            __builtin_amdgcn_sched_barrier(0);
            probe_load<HINT>(r[u], voff, base(i + u + U), i + u + U < cnt);
        });
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const uint32_t x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (x == 0x9e3779b9u) sink[blockIdx.x & 2047] = x;  // (keeps the loads alive; practically never taken)
    clock_record_stop(clk, blockIdx.x == gridDim.x / 2 && threadIdx.x == 0);
}

template<int U>
hipError_t launch_stream(int hint, const void* src, int blocks, void* sink, int grid, hipStream_t st, unsigned long long* clk)
{
    const char* s = (const char*)src;
    uint32_t*   k = (uint32_t*)sink;
    switch (hint) {
        case 0: return launch_kernel(probe_stream_kernel<U, 0>, dim3(grid), dim3(512), 0, st, s, blocks, k, clk);
        case 1: return launch_kernel(probe_stream_kernel<U, 1>, dim3(grid), dim3(512), 0, st, s, blocks, k, clk);
        default: return launch_kernel(probe_stream_kernel<U, 2>, dim3(grid), dim3(512), 0, st, s, blocks, k, clk);
    }
}

// Four independent accumulator chains per wave, operands that change from one MFMA to the next (two fixed
// pseudo-random fragment pairs in turn), `iters` rounds of four MFMAs.
template<int WAVES>
__global__ void __launch_bounds__(64 * WAVES) probe_mfma_kernel(float* sink, int iters, unsigned long long* clk)
{
    clock_record_start(clk, blockIdx.x == gridDim.x / 2 && threadIdx.x == 0);
    half8_t a[2], b[2];
    uint32_t seed = 0x9e3779b9u * (threadIdx.x + 1) + blockIdx.x;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            seed     = seed * 1664525u + 1013904223u;
            a[s][e]  = (half_t)((float)((seed >> 9) & 0xff) * (1.f / 256.f) - 0.5f);
            seed     = seed * 1664525u + 1013904223u;
            b[s][e]  = (half_t)((float)((seed >> 9) & 0xff) * (1.f / 256.f) - 0.5f);
        }
    float4_t acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j & 1], b[(j >> 1) & 1], acc[j], 0, 0, 0);
    }
    const float4_t t = acc[0] + acc[1] + acc[2] + acc[3];
    const float    x = t[0] + t[1] + t[2] + t[3];
    if (x == 12345.678f) sink[blockIdx.x & 2047] = x;  // (keeps the chains alive; practically never taken)
    clock_record_stop(clk, blockIdx.x == gridDim.x / 2 && threadIdx.x == 0);
}

}  // namespace

hipError_t launch_probe_read(const void* src, size_t bytes, void* sink, int cus, hipStream_t st)
{
    const size_t vecs = bytes / 16;
    if (vecs == 0) return hipSuccess;
    const size_t per_pass = (size_t)cus * 512 * 4;
    const int    grid     = (int)std::min<size_t>((vecs + 512 * 4 - 1) / (512 * 4), per_pass ? (size_t)cus * 8 : 1);
    return launch_kernel(probe_read_kernel, dim3(grid), dim3(512), 0, st, (const u32x4_t*)src, vecs, (uint32_t*)sink);
}

bool probe_stream_config_ok(int wg_per_cu, int in_flight, int hint)
{
    return (wg_per_cu == 1 || wg_per_cu == 2 || wg_per_cu == 4) && (in_flight == 2 || in_flight == 4 || in_flight == 8 || in_flight == 16) &&
           hint >= 0 && hint <= 2;
}

hipError_t launch_probe_mfma(void* sink, int cus, int waves_per_cu, int iters, unsigned long long* clk, hipStream_t st)
{
    if (iters < 1 || cus < 1) return hipErrorInvalidValue;
    float* k = (float*)sink;
    switch (waves_per_cu) {
        case 4: return launch_kernel(probe_mfma_kernel<4>, dim3(cus), dim3(256), 0, st, k, iters, clk);
        case 8: return launch_kernel(probe_mfma_kernel<8>, dim3(cus), dim3(512), 0, st, k, iters, clk);
        case 16: return launch_kernel(probe_mfma_kernel<16>, dim3(cus), dim3(1024), 0, st, k, iters, clk);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_probe_stream(const void* src, size_t bytes, void* sink, int cus, int wg_per_cu, int in_flight, int hint,
                               hipStream_t st, unsigned long long* clk)
{
    if (!probe_stream_config_ok(wg_per_cu, in_flight, hint) || bytes / 1024 > (size_t)INT32_MAX) return hipErrorInvalidValue;
    const int blocks = (int)(bytes / 1024);
    if (blocks == 0) return hipSuccess;
    const int grid = cus * wg_per_cu;
    switch (in_flight) {
        case 2: return launch_stream<2>(hint, src, blocks, sink, grid, st, clk);
        case 4: return launch_stream<4>(hint, src, blocks, sink, grid, st, clk);
        case 8: return launch_stream<8>(hint, src, blocks, sink, grid, st, clk);
        default: return launch_stream<16>(hint, src, blocks, sink, grid, st, clk);
    }
}

}  // namespace w4a16
