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

namespace w4a16 {

namespace {

constexpr int kThreads   = 256;
constexpr int kRowHalves = kGroup + 8;  // LDS row stride: 272 bytes, keeps 16 rows on distinct banks

template<int TTILES, int NTW, int EPI>
__global__ void __launch_bounds__(kThreads)
prefill_kernel(uint16_t* __restrict__ C, const u32x4_t* __restrict__ A, const uint16_t* __restrict__ X,
               const uint32_t* __restrict__ Q, const uint16_t* R_, int N, int T, int K, int tiles_t, int tiles_n)
{
    extern __shared__ __attribute__((aligned(16))) uint16_t xs[];  // [2][TT][kRowHalves]
    constexpr int TT   = 16 * TTILES;
    constexpr int TN   = 64 * NTW;
    constexpr int XPER = TTILES / 4;  // 16-byte chunks of X per thread and 32-wide K step

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int c    = lane & 15;
    const int b    = lane >> 4;
    const int G    = K / kGroup;

    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous block of
    // tiles (all token tiles of a few feature tiles) so its private L2 sees the reuse.
    const int total = tiles_t * tiles_n;
    int       id    = blockIdx.x;
    if (total % 8 == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    const int tile_t = id % tiles_t;
    const int tile_n = id / tiles_t;
    const int T0     = tile_t * TT;
    const int nt0    = (tile_n * TN) / kTileN + wave * NTW;  // first weight tile of this wave

    const int64_t   gstride = (int64_t)(N / kTileN) * 64;  // 16-byte units between consecutive groups
    const u32x4_t*  Ap      = A + (int64_t)nt0 * 64 + lane;  // + g * gstride + nt * 64
    const uint32_t* Qp = Q + nt0 * kTileN + c;

    // X staging: chunk (q*256 + tid) -> row q*16 + tid/16, 16-byte column tid%16
    // (rows past the last token re-read the last valid row; their outputs are never stored)
    const int  xr = tid >> 4, xc = tid & 15;
    const auto x_chunk = [&](int q, int g) {
        const int row = min(T0 + q * 16 + xr, T - 1);
        return *reinterpret_cast<const u32x4_t*>(X + (int64_t)row * K + xc * 8 + g * kGroup);
    };
    const int xs_w = xr * kRowHalves + xc * 8;  // + q*16*kRowHalves
    const int xs_r = c * kRowHalves + 8 * b;    // + tt*16*kRowHalves + 32*j

    const UnpackConsts uc;

    float4_t acc[TTILES][NTW];
#pragma unroll
    for (int tt = 0; tt < TTILES; ++tt)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) acc[tt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

    u32x4_t  w[NTW], wn[NTW];
    uint32_t qv[NTW], qn[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        w[nt]  = Ap[nt * 64];
        qv[nt] = Qp[nt * kTileN];
    }
    // first activation tile
#pragma unroll
    for (int q = 0; q < TTILES; ++q) {
        const u32x4_t v = x_chunk(q, 0);
        *reinterpret_cast<u32x4_t*>(&xs[xs_w + q * 16 * kRowHalves]) = v;
    }
    __syncthreads();

    int buf = 0;
    for (int g = 0; g < G; ++g) {
        const bool more = g + 1 < G;
        if (more) {
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
                wn[nt] = Ap[(g + 1) * gstride + nt * 64];
                qn[nt] = Qp[(int64_t)(g + 1) * N + nt * kTileN];
            }
        }
        half2_t z1024[NTW], z64[NTW], sc[NTW];
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            half_t s;
            split_q(qv[nt], z1024[nt], z64[nt], s);
            sc[nt] = half2_t{s, s};
        }
        const uint16_t* xb = xs + buf * (TT * kRowHalves);
        uint16_t*       xo = xs + (buf ^ 1) * (TT * kRowHalves);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            u32x4_t stage[XPER];
            if (more) {
#pragma unroll
                for (int q = 0; q < XPER; ++q)
                    stage[q] = x_chunk(j * XPER + q, g + 1);
            }
            half8_t wf[NTW];
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) wf[nt] = dequant_full(w[nt][j], z1024[nt], z64[nt], sc[nt], uc);
#pragma unroll
            for (int tt = 0; tt < TTILES; ++tt) {
                const half8_t xf =
                    *reinterpret_cast<const half8_t*>(&xb[xs_r + tt * 16 * kRowHalves + 32 * j]);
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt)
                    acc[tt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[nt], xf, acc[tt][nt], 0, 0, 0);
            }
            if (more) {
#pragma unroll
                for (int q = 0; q < XPER; ++q)
                    *reinterpret_cast<u32x4_t*>(&xo[xs_w + (j * XPER + q) * 16 * kRowHalves]) = stage[q];
            }
        }
        __syncthreads();
        buf ^= 1;
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            w[nt]  = wn[nt];
            qv[nt] = qn[nt];
        }
    }

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
constexpr Variant kVariants[] = {{16, 4}, {8, 4}, {16, 2}, {8, 2}, {4, 2}, {4, 1}};
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
        case 0: return launch_v<16, 4>(a, st);
        case 1: return launch_v<8, 4>(a, st);
        case 2: return launch_v<16, 2>(a, st);
        case 3: return launch_v<8, 2>(a, st);
        case 4: return launch_v<4, 2>(a, st);
        default: return launch_v<4, 1>(a, st);
    }
}

}  // namespace w4a16
