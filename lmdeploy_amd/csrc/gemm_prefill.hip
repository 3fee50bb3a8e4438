// Prefill W4A16 GEMM for gfx950: many tokens, bound by the fp16 MFMA rate.
//
// A workgroup of four (or eight) waves computes a (16*TTILES tokens) x (16*NTW*WAVES features)
// output tile.
// The waves split the features; each owns NTW weight tiles per quantisation group and loads
// them straight from global memory into registers (one 128-bit load per lane and tile: the
// tiled layout IS the MFMA operand layout), dequantises them to the reference's exact fp16
// weight fp16_rn((q - z) * s) and uses them as the A operand of v_mfma_f32_16x16x32_f16.
// The activations of the tile go from global memory directly into LDS (no registers, no
// ds_write), double buffered, one 128-wide K step per quantisation group, and are read as the
// B operand by all four waves, so no weight is dequantised twice and no activation is fetched
// twice per workgroup.  With weights as A the accumulator of a lane holds four adjacent
// features of one token, which makes every epilogue (plain, SiLU-gate on feature pairs,
// residual add) lane-local.
//
// The K loop is one hand-scheduled instruction stream per wave: every MFMA is followed by its
// share of the NEXT k32 step's dequantisation, LDS fragment reads and global loads, so that a
// single wave keeps the matrix pipe busy while it issues everything else (measured on this
// part: an MFMA occupies the pipe for 16 cycles and issues in 4; two vector instructions fit
// behind each one for free, a third does not).  The MFMAs are inline assembly with the
// accumulators tied in place in AGPRs; loads are inline assembly waited for by count.
#include "w4a16_common.h"
#include "w4a16_internal.h"

#include <type_traits>

namespace w4a16 {

namespace {

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

// LDS fragment read from inline assembly (byte address + immediate), and its wait.  Left to the
// compiler, each activation fragment was read right before the MFMAs that use it, which then
// waited a full LDS latency; and any compiler-visible LDS read after a direct-to-LDS load would
// be preceded by a wait for ALL loads in flight.  Here the fragments of a k32 step are requested
// during the previous one.
template<int OFF>
__device__ __forceinline__ void lds_read128(half8_t& dst, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
__device__ __forceinline__ void wait_lgkm0(half8_t& a, half8_t& b, half8_t& c, half8_t& d)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

// Register budget: one wave per SIMD (512 registers) for the 128-register accumulator tiles,
// two waves otherwise.  Stating it keeps the allocator from squeezing the kernel into fewer
// VGPRs and parking values in AGPRs, which is fatal here: a register parked while an
// inline-assembly load into it is still in flight is handed to another value, and the load then
// lands on that value (the build rejects kernels that use AGPRs beyond their accumulators).
// WAVES = waves per workgroup (4 or 8), side by side along the features.
template<int TTILES, int NTW, int WAVES, int EPI>
__global__ void __launch_bounds__(64 * WAVES)
    __attribute__((amdgpu_waves_per_eu(TTILES * NTW >= 32 ? 1 : 2, TTILES * NTW >= 32 ? 1 : 2)))
prefill_kernel(uint16_t* __restrict__ C, const u32x4_t* __restrict__ A, const uint16_t* __restrict__ X,
               const uint32_t* __restrict__ Q, const uint16_t* R_, int N, int T, int K, int tiles_t, int tiles_n)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [2][TT][kRowBytes]
    constexpr int TT = 16 * TTILES;
    constexpr int TN = 16 * NTW * WAVES;
    constexpr int XB = 4 * TTILES / WAVES;  // 1 KiB activation blocks (4 token rows) that each wave fetches per group
    static_assert(4 * TTILES % WAVES == 0, "the activation tile must divide evenly among the waves");

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
    // X staging, direct global -> LDS: wave w, request i writes the 1 KiB block m = w*XB + i
    // (token rows 4m .. 4m+3) of the tile; lane l lands at row 4m + l/16, chunk position l%16, so it
    // fetches K-chunk (l%16) ^ (row & 15) of that row.  Rows past the last token re-read the last
    // valid row; their outputs are never stored.
    uint32_t x_off[XB];
#pragma unroll
    for (int i = 0; i < XB; ++i) {
        const int row = 4 * (wave * XB + i) + (lane >> 4);
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
        for (int i = 0; i < XB; ++i) {
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(xbase + x_off[i]),
                (__attribute__((address_space(3))) void*)(xo + (wave * XB + i) * 1024), 16, 0, 0);
        }
    };
    // the same requests one at a time (m = 0 .. 2 NTW + TTILES - 1), to be dealt out between MFMAs
    constexpr int kVmOps = 2 * NTW + XB;
    auto vm_op = [&](auto M, u32x4_t (&w)[NTW], uint32_t (&qv)[NTW], uint8_t* xo, const char* wbase, const char* qbase,
                     const char* xbase) {
        constexpr int m = decltype(M)::value;
        if constexpr (m < NTW) {
            gload128<m * 1024>(w[m], w_off, wbase);
        }
        else if constexpr (m < 2 * NTW) {
            gload32<(m - NTW) * 64>(qv[m - NTW], q_off, qbase);
        }
        else {
            constexpr int i = m - 2 * NTW;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(xbase + x_off[i]),
                (__attribute__((address_space(3))) void*)(xo + (wave * XB + i) * 1024), 16, 0, 0);
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

    // State carried from one k32 step to the next (and across K steps): dequantised weights and
    // activation fragments of the current / next k32 step, zero points and scale of the current /
    // next group.
    half8_t wf[2][NTW];
    half8_t xf[2][TTILES];
    half2_t z1024[2][NTW], z64[2][NTW], sc[2][NTW];

    auto split = [&](auto P_, uint32_t (&qv)[NTW]) {
        constexpr int P = decltype(P_)::value;
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            half_t s;
            split_q(qv[nt], z1024[P][nt], z64[P][nt], s);
            sc[P][nt] = half2_t{s, s};
        }
    };
    // The dequantisation of word J of every tile of `w`, as 13 * NTW single vector instructions
    // (op = NTW * k + nt) so that they can be dealt out between the MFMAs of a k32 step:
    // k = 0: w >> 8;  1..4: (w & mask) | magic;  5..8: - (offset + zero);  9..12: * scale.
    uint32_t dq[NTW][5];
    auto dequant_op = [&](auto P, auto J, auto OP, u32x4_t (&w)[NTW]) {
        constexpr int p = decltype(P)::value, j = decltype(J)::value;
        constexpr int nt = decltype(OP)::value % NTW, k = decltype(OP)::value / NTW;
        if constexpr (k == 0) dq[nt][4] = w[nt][j] >> 8;
        else if constexpr (k <= 4) {
            constexpr int i  = k - 1;
            const uint32_t src = i < 2 ? w[nt][j] : dq[nt][4];
            dq[nt][i] = (src & (i & 1 ? uc.mask_hi : uc.mask_lo)) | (i & 1 ? uc.magic_hi : uc.magic_lo);
        }
        else if constexpr (k <= 8) {
            constexpr int i = k - 5;
            dq[nt][i]       = as_u32(as_half2(dq[nt][i]) - (i & 1 ? z64[p][nt] : z1024[p][nt]));
        }
        else {
            constexpr int i = k - 9;
            const half2_t r = as_half2(dq[nt][i]) * sc[p][nt];
            wf[j & 1][nt][2 * i]     = r[0];
            wf[j & 1][nt][2 * i + 1] = r[1];
        }
    };
    auto dequant = [&](auto P, auto J, u32x4_t (&w)[NTW]) {
        static_for<0, 13 * NTW>([&](auto op) { dequant_op(P, J, op, w); });
    };
    auto read_x = [&](auto J_, const uint8_t* xb) {
        constexpr int  J    = decltype(J_)::value;
        const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)(xb) + xr_off[J];
        static_for<0, TTILES>([&](auto tt) { lds_read128<tt * 16 * kRowBytes>(xf[J & 1][tt], addr); });
    };
    auto read_x1 = [&](auto J_, auto TT_, uint32_t base) {
        constexpr int J = decltype(J_)::value, tt = decltype(TT_)::value;
        lds_read128<tt * 16 * kRowBytes>(xf[J & 1][tt], base + xr_off[J]);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;

    // ---- prologue: groups 0 and 1 in flight, first operands of group 0 prepared ----
    issue_w(wa, qa, 0);
    issue_x(x0, 0);
    issue_w(wb, qb, min(1, G - 1));
    issue_x(x1, min(1, G - 1));
    wait_all(wa, qa);
    wait_all(wb, qb);
    __syncthreads();
    read_x(I0{}, x0);
    split(I0{}, qa);
    dequant(I0{}, I0{}, wa);

    // One K step (a quantisation group, four k32 steps) on the weights `w` (group parity P) and the
    // LDS buffer `xb`.  Every k32 step runs its MFMAs interleaved with the dequantisation of the
    // NEXT k32 step's weights and the requests for its activation fragments.  In the last k32 step
    // the next group's weights (`wn`, requested one K step ago) and activation tile (`xo`) are
    // complete: the workgroup synchronises, starts on them, and re-uses `w` and `xb`, which no wave
    // reads any more, for the loads of group g + 2.
    auto step = [&](auto P, u32x4_t (&w)[NTW], uint32_t (&qv)[NTW], u32x4_t (&wn)[NTW], uint32_t (&qn)[NTW],
                    uint8_t* xb, const uint8_t* xo, int g) {
        constexpr int p  = decltype(P)::value;
        using PN         = std::integral_constant<int, p ^ 1>;
        static_for<0, 4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            using JN        = std::integral_constant<int, (j + 1) & 3>;
#pragma unroll
            for (int tt = 0; tt < TTILES; tt += 4)
                wait_lgkm0(xf[j & 1][tt], xf[j & 1][tt + 1], xf[j & 1][tt + 2], xf[j & 1][tt + 3]);
            const int   g2 = min(g + 2, G - 1);  // (the last steps re-read the last group: no branch)
            const char* wbase = reinterpret_cast<const char*>(A) + (int64_t)g2 * NT * 1024;
            const char* qbase = reinterpret_cast<const char*>(Q) + (int64_t)g2 * N * 4;
            const char* xbase = reinterpret_cast<const char*>(X) + (int64_t)g2 * 256;
            if constexpr (j == 3) {
                wait_all(wn, qn);
                __syncthreads();
            }
            const uint32_t rbase =
                (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)(j < 3 ? (const uint8_t*)xb : xo);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (j == 3) split(PN{}, qn);
            // one MFMA, then its share of the next k32 step's dequantisation, and so on
            constexpr int kOps = 13 * NTW, kSlots = TTILES * NTW;
            static_for<0, kSlots>([&](auto ic) {
                constexpr int i = decltype(ic)::value, tt = i / NTW, nt = i % NTW;
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                             : "+a"(acc[tt][nt])
                             : "v"(wf[j & 1][nt]), "v"(xf[j & 1][tt]));
                __builtin_amdgcn_sched_barrier(0);
                static_for<i * kOps / kSlots, (i + 1) * kOps / kSlots>([&](auto op) {
                    if constexpr (j < 3) dequant_op(P, JN{}, op, w);
                    else dequant_op(PN{}, I0{}, op, wn);
                });
                // the next k32 step's activation fragments, requested during the first three quarters
                // of this one; in the last k32 step also the loads of group g + 2
                constexpr int kR = kSlots * 3 / 4 > 0 ? kSlots * 3 / 4 : 1;
                if constexpr (i < kR) {
                    static_for<i * TTILES / kR, (i + 1) * TTILES / kR>([&](auto tt) { read_x1(JN{}, tt, rbase); });
                }
                if constexpr (j == 3) {
                    static_for<i * kVmOps / kSlots, (i + 1) * kVmOps / kSlots>(
                        [&](auto m) { vm_op(m, w, qv, xb, wbase, qbase, xbase); });
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };

    int g = 0;
    for (; g + 1 < G; g += 2) {  // no branch inside: the 4*TTILES*NTW accumulators stay in place
        step(I0{}, wa, qa, wb, qb, x0, x1, g);
        step(I1{}, wb, qb, wa, qa, x1, x0, g + 1);
    }
    if (g < G) step(I0{}, wa, qa, wb, qb, x0, x1, g);
    wait_all(wa, qa);  // no load may still be writing LDS or registers when the wave ends
    wait_all(wb, qb);
    // the MFMAs are inline assembly, so the compiler does not know that the accumulators are
    // still being written: cover the longest MFMA-result-to-VALU-read distance by hand
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

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
    int ttiles, ntw, waves;
};
// (a 256 x 256 tile does not fit the register file without spilling, and spill stores would
// break the counted waits: stores and loads complete out of order with each other)
// (first match wins in the dispatcher: the 8-wave 128 x 256 tile comes before the 4-wave one)
constexpr Variant kVariants[] = {{8, 2, 8}, {16, 2, 4}, {8, 2, 4}, {4, 2, 4}, {4, 1, 4}, {8, 4, 4}};
constexpr int     kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template<int TTILES, int NTW, int WAVES>
hipError_t launch_v(const GemmArgs& a, hipStream_t st)
{
    constexpr int TT = 16 * TTILES, TN = 16 * NTW * WAVES;
    const int     tiles_t = (a.T + TT - 1) / TT;
    const int     tiles_n = a.N / TN;
    const size_t  lds     = (size_t)2 * TT * kRowBytes;
    const dim3    grid(tiles_t * tiles_n), block(64 * WAVES);
    const u32x4_t* A4 = reinterpret_cast<const u32x4_t*>(a.A);
#define W4A16_LAUNCH(EPI)                                                                                              \
    do {                                                                                                               \
        auto       kfn = prefill_kernel<TTILES, NTW, WAVES, EPI>;                                                             \
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
    tile_n = 16 * kVariants[v].ntw * kVariants[v].waves;
    tile_t = 16 * kVariants[v].ttiles;
}

bool prefill_feasible(int v, int N, int T, int K)
{
    if (v < 0 || v >= kNumVariants || N <= 0 || T <= 0 || K <= 0) return false;
    const int tn = 16 * kVariants[v].ntw * kVariants[v].waves, tt = 16 * kVariants[v].ttiles;
    if (N % tn != 0 || K % kGroup != 0) return false;
    // per-thread offsets into X and into one group of A are 32-bit
    if ((int64_t)T * K * 2 >= (1ll << 32) || (int64_t)N * 64 >= (1ll << 32)) return false;
    const int64_t grid = (int64_t)(N / tn) * ((T + tt - 1) / tt);
    return grid < (1ll << 31);
}

int prefill_grid(int v, int N, int T, int K)
{
    (void)K;
    const int tn = 16 * kVariants[v].ntw * kVariants[v].waves, tt = 16 * kVariants[v].ttiles;
    return (N / tn) * ((T + tt - 1) / tt);
}

hipError_t prefill_launch(int v, const GemmArgs& a, hipStream_t st)
{
    switch (v) {
        case 0: return launch_v<8, 2, 8>(a, st);
        case 1: return launch_v<16, 2, 4>(a, st);
        case 2: return launch_v<8, 2, 4>(a, st);
        case 3: return launch_v<4, 2, 4>(a, st);
        case 4: return launch_v<4, 1, 4>(a, st);
        default: return launch_v<8, 4, 4>(a, st);
    }
}

}  // namespace w4a16
