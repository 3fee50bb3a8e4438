// Prefill W4A16 GEMM for gfx950: many tokens, bound by the fp16 MFMA rate.
//
// A workgroup of four waves computes a (16*TTILES tokens) x (64*NTW features) output tile.
// The waves split the features; each owns NTW weight tiles per quantisation group and loads
// them straight from global memory into registers (one 128-bit load per lane and tile: the
// tiled layout IS the MFMA operand layout), dequantises them to the reference's exact fp16
// weight fp16_rn((q - z) * s) and uses them as the A operand of v_mfma_f32_16x16x32_f16.
// The activations of the tile are staged once per workgroup in LDS (double buffered, one
// 128-wide K step per quantisation group) and read as the B operand by all four waves, so
// no weight is dequantised twice and no activation is fetched twice per workgroup.
// With weights as A the accumulator of a lane holds four adjacent features of one token,
// which makes every epilogue (plain, SiLU-gate on feature pairs, residual add) lane-local.
#include "w4a16_common.h"
#include "w4a16_internal.h"

#include <type_traits>

namespace w4a16 {

namespace {

constexpr int kThreads   = 256;
#ifndef W4A16_ROWPAD
#define W4A16_ROWPAD 16
#endif
constexpr int kRowHalves = kGroup + W4A16_ROWPAD;  // LDS row stride 288 bytes: measured free of bank conflicts (272 is not)

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(<N-1>); gives inline assembly
// its immediate operands.
template<int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Loads of the software pipeline.  They are issued from inline assembly, in place ("+v"), with
// a scalar base and a per-thread 32-bit offset, and waited for by count: the compiler would
// drain every load in flight at the loop header, exposing the memory latency once per K step.
template<int OFF>
__device__ __forceinline__ void gload128(u32x4_t& dst, uint32_t voff, const void* sbase)
{
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(OFF));
}
template<int OFF>
__device__ __forceinline__ void gload32(uint32_t& dst, uint32_t voff, const void* sbase)
{
    asm volatile("global_load_dword %0, %1, %2 offset:%3" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(OFF));
}
// wait until at most N of this wave's loads are in flight; tied to `v` so that no use of it can
// be scheduled above the wait
template<int N, typename V>
__device__ __forceinline__ void wait_vm(V& v)
{
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(v) : "n"(N));
}

// Register budget: one wave per SIMD (512 registers) for the 256-register accumulator tiles,
// two waves otherwise.  Stating it keeps the allocator from squeezing the kernel into fewer
// VGPRs and shuttling values through AGPRs inside the loop.
template<int TTILES, int NTW, int EPI>
__global__ void __launch_bounds__(kThreads)
    __attribute__((amdgpu_waves_per_eu(TTILES * NTW >= 32 ? 1 : 2, TTILES * NTW >= 32 ? 1 : 2)))
prefill_kernel(uint16_t* __restrict__ C, const u32x4_t* __restrict__ A, const uint16_t* __restrict__ X,
               const uint32_t* __restrict__ Q, const uint16_t* R_, int N, int T, int K, int tiles_t, int tiles_n)
{
    extern __shared__ __attribute__((aligned(16))) uint16_t xs[];  // [2][TT][kRowHalves]
    constexpr int TT = 16 * TTILES;
    constexpr int TN = 64 * NTW;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c    = lane & 15;
    const int b    = lane >> 4;
    const int G    = K / kGroup;
    const int NT   = N / kTileN;

    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of tiles so
    // its private L2 sees the reuse.  Inside a run, tiles go four token tiles at a time across
    // the feature tiles: the ~64 workgroups an XCD runs concurrently then cover 4 token tiles x
    // 16 feature tiles, which minimises what they fetch together (a token tile of activations
    // is four times larger than a feature tile of int4 weights).
    const int total = tiles_t * tiles_n;
    int       id    = blockIdx.x;
    if (total % 8 == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    int tile_t, tile_n;
    if (tiles_t % 4 == 0) {
        const int r = id >> 2;
        tile_n      = r % tiles_n;
        tile_t      = (r / tiles_n) * 4 + (id & 3);
    }
    else {
        tile_t = id % tiles_t;
        tile_n = id / tiles_t;
    }
    const int T0     = tile_t * TT;
    const int nt0    = (tile_n * TN) / kTileN + wave * NTW;  // first weight tile of this wave

    // per-thread byte offsets; the group-dependent part of every address is scalar
    const uint32_t w_off = (uint32_t)(nt0 * 1024 + lane * 16);        // + g * NT * 1024 (+ nt * 1024)
    const uint32_t q_off = (uint32_t)((nt0 * kTileN + c) * 4);        // + g * N * 4    (+ nt * 64)
    // X staging: chunk q of this thread is row q*16 + tid/16, 16-byte column tid%16 of the tile
    // (rows past the last token re-read the last valid row; their outputs are never stored)
    const int xr = tid >> 4, xc = tid & 15;
    uint32_t  x_off[TTILES];
#pragma unroll
    for (int q = 0; q < TTILES; ++q)
        x_off[q] = (uint32_t)(min(T0 + q * 16 + xr, T - 1)) * (uint32_t)(K * 2) + xc * 16;  // + g * 256
    const int xs_w = xr * kRowHalves + xc * 8;  // + q*16*kRowHalves
    const int xs_r = c * kRowHalves + 8 * b;    // + tt*16*kRowHalves + 32*j

    const UnpackConsts uc;

    float4_t acc[TTILES][NTW];
#pragma unroll
    for (int tt = 0; tt < TTILES; ++tt)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) acc[tt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

    u32x4_t  wa[NTW], wb[NTW];  // weights of the current / next group (roles alternate)
    uint32_t qa[NTW], qb[NTW];
    constexpr int XB = TTILES < 8 ? TTILES : 8;  // activation chunks staged at a time
    u32x4_t       xst[XB];                        // activations of the next group on their way to LDS
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        wa[nt] = wb[nt] = u32x4_t{0, 0, 0, 0};
        qa[nt] = qb[nt] = 0;
    }
#pragma unroll
    for (int q = 0; q < XB; ++q) xst[q] = u32x4_t{0, 0, 0, 0};

    auto issue_w = [&](u32x4_t (&w)[NTW], uint32_t (&qv)[NTW], int g) {
        const char* wbase = reinterpret_cast<const char*>(A) + (int64_t)g * NT * 1024;
        const char* qbase = reinterpret_cast<const char*>(Q) + (int64_t)g * N * 4;
        static_for<0, NTW>([&](auto nt) { gload128<nt * 1024>(w[nt], w_off, wbase); });
        static_for<0, NTW>([&](auto nt) { gload32<nt * 64>(qv[nt], q_off, qbase); });
    };
    // activation chunks [q0, q0 + XB) of group g: request, and (later) wait for all and store
    auto issue_x = [&](int q0, int g) {
        const char* xbase = reinterpret_cast<const char*>(X) + (int64_t)g * 256;
#pragma unroll
        for (int q = 0; q < XB; ++q) gload128<0>(xst[q], x_off[q0 + q], xbase);
    };
    auto store_x = [&](uint16_t* xo, int q0) {
#pragma unroll
        for (int q = 0; q < XB; ++q) {
            wait_vm<0>(xst[q]);
            *reinterpret_cast<u32x4_t*>(&xo[xs_w + (q0 + q) * 16 * kRowHalves]) = xst[q];
        }
    };

    // ---- prologue: group 0 ----
    issue_w(wa, qa, 0);
#pragma unroll
    for (int q0 = 0; q0 < TTILES; q0 += XB) {
        issue_x(q0, 0);
        store_x(xs, q0);
    }
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        wait_vm<0>(wa[nt]);
        wait_vm<0>(qa[nt]);
    }
    __syncthreads();

    // One K step (a quantisation group): MFMAs on `w`/buffer `xb` while the next group's
    // weights go to `wn` and its activations to the other LDS buffer `xo`.
    auto step = [&](u32x4_t (&w)[NTW], uint32_t (&qv)[NTW], u32x4_t (&wn)[NTW], uint32_t (&qn)[NTW],
                    const uint16_t* xb, uint16_t* xo, int g) {
        const int gn = min(g + 1, G - 1);  // (the last step re-reads its own group: no branch)
        issue_w(wn, qn, gn);
        issue_x(0, gn);
        half2_t z1024[NTW], z64[NTW], sc[NTW];
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            half_t s;
            split_q(qv[nt], z1024[nt], z64[nt], s);
            sc[nt] = half2_t{s, s};
        }
        static_for<0, 4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            half8_t       wf[NTW];
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) wf[nt] = dequant_full(w[nt][j], z1024[nt], z64[nt], sc[nt], uc);
#pragma unroll
            for (int tt = 0; tt < TTILES; ++tt) {
                const half8_t xf = *reinterpret_cast<const half8_t*>(&xb[xs_r + tt * 16 * kRowHalves + 32 * j]);
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt)
                    acc[tt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[nt], xf, acc[tt][nt], 0, 0, 0);
            }
            // staged activations: with 16 token tiles the first 8 chunks are stored (and the other
            // 8 requested) after the second k32 step; the last batch is stored after the fourth
            if constexpr (TTILES > XB && j == 1) {
                store_x(xo, 0);
                issue_x(XB, gn);
            }
            if constexpr (j == 3) store_x(xo, TTILES - XB);
        });
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {  // everything has landed (vmcnt(0) above); pin the uses below it
            wait_vm<0>(wn[nt]);
            wait_vm<0>(qn[nt]);
        }
        __syncthreads();
    };

    uint16_t* const x0 = xs;
    uint16_t* const x1 = xs + TT * kRowHalves;
    int g = 0;
    for (; g + 1 < G; g += 2) {  // no branch inside: the 4*TTILES*NTW accumulators stay in place
        step(wa, qa, wb, qb, x0, x1, g);
        step(wb, qb, wa, qa, x1, x0, g + 1);
    }
    if (g < G) step(wa, qa, wb, qb, x0, x1, g);

    // ---- epilogue: lane (c, b) of tile (tt, nt) holds token T0 + 16 tt + c, features n .. n+3 ----
#pragma unroll
    for (int tt = 0; tt < TTILES; ++tt) {
        const int token = T0 + tt * 16 + c;
        if (token >= T) continue;
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            const int      n = (nt0 + nt) * kTileN + 4 * b;
            const float4_t v = acc[tt][nt];
            const half_t   h0 = (half_t)v[0], h1 = (half_t)v[1], h2 = (half_t)v[2], h3 = (half_t)v[3];
            if constexpr (EPI == kEpiGemm) {
                uint2 o;
                o.x = as_u32(half2_t{h0, h1});
                o.y = as_u32(half2_t{h2, h3});
                *reinterpret_cast<uint2*>(C + (int64_t)token * N + n) = o;
            }
            else if constexpr (EPI == kEpiSilu) {
                const float  g0 = (float)h0, u0 = (float)h1, g1 = (float)h2, u1 = (float)h3;
                const half_t o0 = (half_t)(g0 / (1.f + __expf(-g0)) * u0);
                const half_t o1 = (half_t)(g1 / (1.f + __expf(-g1)) * u1);
                *reinterpret_cast<uint32_t*>(C + (int64_t)token * (N / 2) + (n >> 1)) = as_u32(half2_t{o0, o1});
            }
            else {
                const uint2   rr = *reinterpret_cast<const uint2*>(R_ + (int64_t)token * N + n);
                const half2_t r0 = as_half2(rr.x), r1 = as_half2(rr.y);
                uint2         o;
                o.x = as_u32(half2_t{(half_t)((float)r0[0] + (float)h0), (half_t)((float)r0[1] + (float)h1)});
                o.y = as_u32(half2_t{(half_t)((float)r1[0] + (float)h2), (half_t)((float)r1[1] + (float)h3)});
                *reinterpret_cast<uint2*>(C + (int64_t)token * N + n) = o;
            }
        }
    }
}

struct Variant {
    int ttiles, ntw;
};
// (a 256 x 256 tile does not fit the register file without spilling, and spill stores would
// break the counted waits: stores and loads complete out of order with each other)
constexpr Variant kVariants[] = {{8, 4}, {16, 2}, {8, 2}, {4, 2}, {4, 1}};
constexpr int     kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template<int TTILES, int NTW>
hipError_t launch_v(const GemmArgs& a, hipStream_t st)
{
    constexpr int TT = 16 * TTILES, TN = 64 * NTW;
    const int     tiles_t = (a.T + TT - 1) / TT;
    const int     tiles_n = a.N / TN;
    const size_t  lds     = (size_t)2 * TT * kRowHalves * sizeof(uint16_t);
    const dim3    grid(tiles_t * tiles_n), block(kThreads);
    const u32x4_t* A4 = reinterpret_cast<const u32x4_t*>(a.A);
#define W4A16_LAUNCH(EPI)                                                                                              \
    do {                                                                                                               \
        auto       kfn = prefill_kernel<TTILES, NTW, EPI>;                                                             \
        hipError_t e   = hipFuncSetAttribute(reinterpret_cast<const void*>(kfn),                                       \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                     \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kfn, grid, block, lds, st, a.C, A4, a.X, a.Q, a.R, a.N, a.T, a.K, tiles_t, tiles_n);        \
    } while (0)
    switch (a.epilogue) {
        case kEpiGemm: W4A16_LAUNCH(kEpiGemm); break;
        case kEpiSilu: W4A16_LAUNCH(kEpiSilu); break;
        default: W4A16_LAUNCH(kEpiAdd); break;
    }
#undef W4A16_LAUNCH
    return hipGetLastError();
}

}  // namespace

int prefill_variants()
{
    return kNumVariants;
}

void prefill_tile(int v, int& tile_n, int& tile_t)
{
    tile_n = 64 * kVariants[v].ntw;
    tile_t = 16 * kVariants[v].ttiles;
}

bool prefill_feasible(int v, int N, int T, int K)
{
    if (v < 0 || v >= kNumVariants || N <= 0 || T <= 0 || K <= 0) return false;
    const int tn = 64 * kVariants[v].ntw, tt = 16 * kVariants[v].ttiles;
    if (N % tn != 0 || K % kGroup != 0) return false;
    // per-thread offsets into X and into one group of A are 32-bit
    if ((int64_t)T * K * 2 >= (1ll << 32) || (int64_t)N * 64 >= (1ll << 32)) return false;
    const int64_t grid = (int64_t)(N / tn) * ((T + tt - 1) / tt);
    return grid < (1ll << 31);
}

int prefill_grid(int v, int N, int T, int K)
{
    (void)K;
    const int tn = 64 * kVariants[v].ntw, tt = 16 * kVariants[v].ttiles;
    return (N / tn) * ((T + tt - 1) / tt);
}

hipError_t prefill_launch(int v, const GemmArgs& a, hipStream_t st)
{
    switch (v) {
        case 0: return launch_v<8, 4>(a, st);
        case 1: return launch_v<16, 2>(a, st);
        case 2: return launch_v<8, 2>(a, st);
        case 3: return launch_v<4, 2>(a, st);
        default: return launch_v<4, 1>(a, st);
    }
}

}  // namespace w4a16
