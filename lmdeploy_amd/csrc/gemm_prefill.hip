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
// LDS holds two activation tiles of [tokens][128 halves] = 256 bytes per token row, i.e. 16 chunks
// of 16 bytes.  Chunk position p of row r holds K-chunk p ^ (r & 15): the 16 lanes that read the
// same K-chunk of 16 consecutive rows then hit 16 different bank groups, without padding, which
// the direct global-to-LDS loads (64 lanes x 16 contiguous bytes) could not produce.
constexpr int kRowBytes = kGroup * 2;

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
// LDS fragment read from inline assembly (byte address + immediate), and its wait.  Left to the
// compiler, each activation fragment was read right before the two MFMAs that use it, so every
// pair of MFMAs (32 cycles of matrix work) waited a full LDS latency.  Here a whole k32 step of
// fragments is requested one step ahead.
template<int OFF>
__device__ __forceinline__ void lds_read128(half8_t& dst, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
__device__ __forceinline__ void wait_lgkm0(half8_t& v)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v));
}

template<int TTILES, int NTW, int EPI>
__global__ void __launch_bounds__(kThreads)
    __attribute__((amdgpu_waves_per_eu(TTILES * NTW >= 32 ? 1 : 2, TTILES * NTW >= 32 ? 1 : 2)))
prefill_kernel(uint16_t* __restrict__ C, const u32x4_t* __restrict__ A, const uint16_t* __restrict__ X,
               const uint32_t* __restrict__ Q, const uint16_t* R_, int N, int T, int K, int tiles_t, int tiles_n)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [2][TT][kRowBytes]
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
    // X staging, direct global -> LDS: wave w, request i writes the 1 KiB block m = w*TTILES + i
    // (token rows 4m .. 4m+3) of the tile; lane l lands at row 4m + l/16, chunk position l%16, so it
    // fetches K-chunk (l%16) ^ (row & 15) of that row.  Rows past the last token re-read the last
    // valid row; their outputs are never stored.
    uint32_t x_off[TTILES];
#pragma unroll
    for (int i = 0; i < TTILES; ++i) {
        const int row = 4 * (wave * TTILES + i) + (lane >> 4);
        x_off[i] = (uint32_t)min(T0 + row, T - 1) * (uint32_t)(K * 2) + (uint32_t)(((lane & 15) ^ (row & 15)) * 16);
    }
    // fragment reads: lane (c, b) reads row 16*tt + c, K-chunk 4j + b  ->  position (4j + b) ^ c
    uint32_t xr_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) xr_off[j] = (uint32_t)(c * kRowBytes + (((4 * j + b) ^ c) & 15) * 16);

    const UnpackConsts uc;

    float4_t acc[TTILES][NTW];
#pragma unroll
    for (int tt = 0; tt < TTILES; ++tt)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) acc[tt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

    u32x4_t  wa[NTW], wb[NTW];  // weights of the current / next group (roles alternate)
    uint32_t qa[NTW], qb[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        wa[nt] = wb[nt] = u32x4_t{0, 0, 0, 0};
        qa[nt] = qb[nt] = 0;
    }

    auto issue_w = [&](u32x4_t (&w)[NTW], uint32_t (&qv)[NTW], int g) {
        const char* wbase = reinterpret_cast<const char*>(A) + (int64_t)g * NT * 1024;
        const char* qbase = reinterpret_cast<const char*>(Q) + (int64_t)g * N * 4;
        static_for<0, NTW>([&](auto nt) { gload128<nt * 1024>(w[nt], w_off, wbase); });
        static_for<0, NTW>([&](auto nt) { gload32<nt * 64>(qv[nt], q_off, qbase); });
    };
    // the activation tile of group g, straight into the LDS buffer `xo` (no registers, no ds_write)
    auto issue_x = [&](uint8_t* xo, int g) {
        const char* xbase = reinterpret_cast<const char*>(X) + (int64_t)g * 256;
#pragma unroll
        for (int i = 0; i < TTILES; ++i) {
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(xbase + x_off[i]),
                (__attribute__((address_space(3))) void*)(xo + (wave * TTILES + i) * 1024), 16, 0, 0);
        }
    };
    auto wait_all = [&](u32x4_t (&w)[NTW], uint32_t (&qv)[NTW]) {
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            wait_vm<0>(w[nt]);
            wait_vm<0>(qv[nt]);
        }
    };

    uint8_t* const x0 = xs;
    uint8_t* const x1 = xs + TT * kRowBytes;

    // ---- prologue: group 0 ----
    issue_w(wa, qa, 0);
    issue_x(x0, 0);
    wait_all(wa, qa);
    __syncthreads();

    // One K step (a quantisation group): MFMAs on `w`/buffer `xb` while the next group's
    // weights go to `wn` and its activations to the other LDS buffer `xo`.
    auto step = [&](u32x4_t (&w)[NTW], uint32_t (&qv)[NTW], u32x4_t (&wn)[NTW], uint32_t (&qn)[NTW],
                    const uint8_t* xb, uint8_t* xo, int g) {
        const int gn = min(g + 1, G - 1);  // (the last step re-reads its own group: no branch)
        issue_w(wn, qn, gn);
        issue_x(xo, gn);
        half2_t z1024[NTW], z64[NTW], sc[NTW];
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            half_t s;
            split_q(qv[nt], z1024[nt], z64[nt], s);
            sc[nt] = half2_t{s, s};
        }
        // byte address in LDS of the tile being read
        const uint32_t xb_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)(xb);
        half8_t        xf[2][TTILES];  // fragments of the current / next k32 step
        static_for<0, TTILES>([&](auto tt) { lds_read128<tt * 16 * kRowBytes>(xf[0][tt], xb_addr + xr_off[0]); });
        static_for<0, 4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            half8_t       wf[NTW];
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) wf[nt] = dequant_full(w[nt][j], z1024[nt], z64[nt], sc[nt], uc);
#pragma unroll
            for (int tt = 0; tt < TTILES; ++tt) wait_lgkm0(xf[j & 1][tt]);
            if constexpr (j < 3) {
                static_for<0, TTILES>([&](auto tt) {
                    lds_read128<tt * 16 * kRowBytes>(xf[(j + 1) & 1][tt], xb_addr + xr_off[j + 1]);
                });
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the requests above this step's MFMAs
#pragma unroll
            for (int tt = 0; tt < TTILES; ++tt) {
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt)
                    acc[tt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[nt], xf[j & 1][tt], acc[tt][nt], 0, 0, 0);
            }
        });
        // next group's weights are in registers and its activations in LDS once every load of this
        // wave has completed; the barrier then publishes the other waves' parts of the tile
        wait_all(wn, qn);
        __syncthreads();
    };

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
    const size_t  lds     = (size_t)2 * TT * kRowBytes;
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
